// The tile quantizer for 2-, 3-, 5- and 6-bit codes (kvhip_quant_tile.hpp), in a translation unit of its own.
#include "kvhip_quant_tile.hpp"

namespace kvhip {

hipError_t launch_quant_tiles_other(const Store &st, const void *keys, const void *values, int L, int a0, int b0, int tiles,
                                    hipStream_t s, const RopeDev &r) {
    switch (st.bits) {
    case 2: return launch_quant_tiles_bits<2, false, false>(st, st, keys, values, L, a0, b0, tiles, s, r);
    case 3: return launch_quant_tiles_bits<3, false, false>(st, st, keys, values, L, a0, b0, tiles, s, r);
    case 5: return launch_quant_tiles_bits<5, false, false>(st, st, keys, values, L, a0, b0, tiles, s, r);
    case 6: return launch_quant_tiles_bits<6, false, false>(st, st, keys, values, L, a0, b0, tiles, s, r);
    }
    return hipErrorInvalidValue;
}

hipError_t launch_requant_tiles_other(const Store &src, const Store &st, int tiles, hipStream_t s) {
    const RopeDev none;
    switch (st.bits) {
    case 2: return launch_quant_tiles_bits<2, false, true>(st, src, nullptr, nullptr, 0, 0, 0, tiles, s, none);
    case 3: return launch_quant_tiles_bits<3, false, true>(st, src, nullptr, nullptr, 0, 0, 0, tiles, s, none);
    case 5: return launch_quant_tiles_bits<5, false, true>(st, src, nullptr, nullptr, 0, 0, 0, tiles, s, none);
    case 6: return launch_quant_tiles_bits<6, false, true>(st, src, nullptr, nullptr, 0, 0, 0, tiles, s, none);
    }
    return hipErrorInvalidValue;
}

}  // namespace kvhip
