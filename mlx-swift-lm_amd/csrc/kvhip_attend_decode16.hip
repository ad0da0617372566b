// The 16-row split-sequence kernel (kvhip_attend_decode16.hpp) for 4- and 8-bit codes, and which shapes the other code
// widths have instances for.
#include "kvhip_attend_decode16.hpp"

namespace kvhip {

// 2-, 3-, 5- and 6-bit codes: equal head sizes of 64 (groups of 32 / 64), 96 (32), 128 (32 / 64 / 128) and 256 (64),
// keys of 192 with values of 128 (64)
bool decode16_stream_shape(const Store &s) {
    if (s.bits != 2 && s.bits != 3 && s.bits != 5 && s.bits != 6) return false;
    if (s.Dk == 192 && s.Dv == 128) return s.gs == 64;
    if (s.Dk != s.Dv) return false;
    if (s.Dk == 64) return s.gs == 32 || s.gs == 64;
    if (s.Dk == 96) return s.gs == 32;
    if (s.Dk == 128) return s.gs == 32 || s.gs == 64 || s.gs == 128;
    if (s.Dk == 256) return s.gs == 64;
    return false;
}

hipError_t launch_attend_decode16(const AttendArgs &a, int tiles_total, int tiles_per_wg, int nsplit, hipStream_t s) {
    switch (a.st.bits) {
    case 4: return launch_decode16_bits<4>(a, tiles_total, tiles_per_wg, nsplit, s);
    case 8: return launch_decode16_bits<8>(a, tiles_total, tiles_per_wg, nsplit, s);
    case 2:
    case 3: return launch_attend_decode16_low(a, tiles_total, tiles_per_wg, nsplit, s);
    case 5:
    case 6: return launch_attend_decode16_high(a, tiles_total, tiles_per_wg, nsplit, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace kvhip
