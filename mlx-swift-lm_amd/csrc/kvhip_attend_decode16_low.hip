// The 16-row split-sequence kernel (kvhip_attend_decode16.hpp) for 2- and 3-bit codes.
#include "kvhip_attend_decode16.hpp"

namespace kvhip {

hipError_t launch_attend_decode16_low(const AttendArgs &a, int tiles_total, int tiles_per_wg, int nsplit, hipStream_t s) {
    if (a.st.bits == 2) return launch_decode16_bits<2>(a, tiles_total, tiles_per_wg, nsplit, s);
    return launch_decode16_bits<3>(a, tiles_total, tiles_per_wg, nsplit, s);
}

}  // namespace kvhip
