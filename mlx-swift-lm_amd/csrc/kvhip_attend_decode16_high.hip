// The 16-row split-sequence kernel (kvhip_attend_decode16.hpp) for 5- and 6-bit codes.
#include "kvhip_attend_decode16.hpp"

namespace kvhip {

hipError_t launch_attend_decode16_high(const AttendArgs &a, int tiles_total, int tiles_per_wg, int nsplit, hipStream_t s) {
    if (a.st.bits == 5) return launch_decode16_bits<5>(a, tiles_total, tiles_per_wg, nsplit, s);
    return launch_decode16_bits<6>(a, tiles_total, tiles_per_wg, nsplit, s);
}

}  // namespace kvhip
