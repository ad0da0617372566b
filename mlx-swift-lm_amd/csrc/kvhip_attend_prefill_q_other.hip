// The pipelined prefill tile for quantized caches (kvhip_attend_prefill_q.hpp): 2-, 3-, 5- and 6-bit codes (more than
// 16 query rows per kv head, and every row count of the shapes the 16-row decode kernel has no instance for).
#include "kvhip_attend_prefill_q.hpp"

namespace kvhip {

hipError_t launch_attend_prefill_q_other(const AttendArgs &a, int nsplit, int rows, hipStream_t s) {
    switch (a.st.bits) {
    case 2: return launch_prefill_q_bits<2, false>(a, nsplit, rows, s);
    case 3: return launch_prefill_q_bits<3, false>(a, nsplit, rows, s);
    case 5: return launch_prefill_q_bits<5, false>(a, nsplit, rows, s);
    case 6: return launch_prefill_q_bits<6, false>(a, nsplit, rows, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace kvhip
