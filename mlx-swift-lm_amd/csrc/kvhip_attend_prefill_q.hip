// The pipelined prefill tile for quantized caches (kvhip_attend_prefill_q.hpp): 4- and 8-bit codes, and the entry
// points of all code widths.
#include "kvhip_attend_prefill_q.hpp"

namespace kvhip {

bool attend_prefill_q_supported(const AttendArgs &a) {
    const Store &s = a.st;
    if (s.dtype != KVHIP_F16 && s.dtype != KVHIP_BF16) return false;
    if (s.bits != 2 && s.bits != 3 && s.bits != 4 && s.bits != 5 && s.bits != 6 && s.bits != 8) return false;
    // one head size for keys and values, or keys of 192 with values of 128 (the multi-head latent attention models)
    const bool same = s.Dk == s.Dv && (s.Dk == 64 || s.Dk == 96 || s.Dk == 128 || s.Dk == 256);
    if (!same && !(s.Dk == 192 && s.Dv == 128)) return false;
    if (s.gs < 32 || s.Dk % s.gs != 0 || s.Dv % s.gs != 0 || s.Dv / s.gs > 8) return false;
    return a.runs.n == 1 && a.runs.row0[0] == 0 && a.runs.phys0[0] == 0;  // slots in presented order
}

hipError_t launch_attend_prefill_q(const AttendArgs &a, int nsplit, int rows, hipStream_t s) {
    if (a.st.bits == 4) return launch_prefill_q_bits<4, true>(a, nsplit, rows, s);
    if (a.st.bits == 8) return launch_prefill_q_bits<8, true>(a, nsplit, rows, s);
    return launch_attend_prefill_q_other(a, nsplit, rows, s);
}

}  // namespace kvhip
