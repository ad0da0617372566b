// Mask evaluation shared by the attention kernels.
#pragma once
#include "kvhip_device.hpp"

namespace kvhip {

// Decides whether query row l (of L) of batch b / query head hq may see presented
// key row j (of T).  `add` receives the additive term of a float array mask.
__device__ __forceinline__ bool mask_keep(const MaskDev &m, int b, int hq, int l, int j, int L, int T,
                                          float &add) {
    add = 0.0f;
    switch (m.mode) {
        case KVHIP_MASK_CAUSAL:
            return j <= T - L + l;
        case KVHIP_MASK_ARRAY: {
            const size_t i = (size_t)(b * m.sb + hq * m.sh + l * m.sl) + j;
            if (m.dtype == KVHIP_BOOL) return reinterpret_cast<const uint8_t *>(m.data)[i] != 0;
            if (m.dtype == KVHIP_F16) add = Elem<0>::load(m.data, i);
            else if (m.dtype == KVHIP_BF16) add = Elem<1>::load(m.data, i);
            else add = Elem<2>::load(m.data, i);
            return true;
        }
        case KVHIP_MASK_WINDOW: {
            const int li = m.offset + l;
            bool keep = li >= j;
            if (m.window > 0) keep = keep && (li < j + m.window);
            if (m.lengths) keep = keep && (j < m.lengths[b]);
            if (m.left_pad) keep = keep && (j >= m.left_pad[b]);
            return keep;
        }
        default:
            return true;
    }
}

// 4 * W consecutive bytes of a boolean array mask: query row l of (b, hq), key rows j0 .. j0 + 4 W - 1
// (all below T; the address need not be aligned: global loads take any byte address).  One
// load in place of 4 W byte loads per lane.
template <int W>
__device__ __forceinline__ void mask_bool_words(const MaskDev &m, int b, int hq, int l, int j0, uint32_t (&w)[W]) {
    const uint8_t *p = reinterpret_cast<const uint8_t *>(m.data) + (size_t)(b * m.sb + hq * m.sh + l * m.sl) + j0;
    struct __attribute__((packed, aligned(1))) Raw {
        uint32_t v[W];
    };
    const Raw raw = *reinterpret_cast<const Raw *>(p);
#pragma unroll
    for (int i = 0; i < W; ++i) w[i] = raw.v[i];
}

// Index-only masks (causal, window with optional per-batch bounds) with the per-batch
// bounds already in registers: no memory access, so kernels can keep loads in flight.
struct SymMask {
    int mode, offset, window, len_b, pad_b, T, L;
};
__device__ __forceinline__ SymMask sym_mask_init(const MaskDev &m, int b, int L, int T) {
    SymMask s;
    s.mode = m.mode;
    s.offset = m.offset;
    s.window = m.window;
    s.len_b = (m.mode == KVHIP_MASK_WINDOW && m.lengths) ? m.lengths[b] : 0x7fffffff;
    s.pad_b = (m.mode == KVHIP_MASK_WINDOW && m.left_pad) ? m.left_pad[b] : 0;
    s.T = T;
    s.L = L;
    return s;
}
__device__ __forceinline__ bool sym_mask_keep(const SymMask &s, int l, int j) {
    if (s.mode == KVHIP_MASK_CAUSAL) return j <= s.T - s.L + l;
    const int li = s.offset + l;
    bool keep = li >= j && j < s.len_b && j >= s.pad_b;
    if (s.window > 0) keep = keep && (li < j + s.window);
    return keep;
}

// Inclusive range of key rows any query position l in [0, L) may see under an index-only mask.
__device__ __forceinline__ void sym_mask_row_range(const SymMask &s, int &lo, int &hi) {
    if (s.mode == KVHIP_MASK_CAUSAL) {
        lo = 0;
        hi = s.T - 1;
        return;
    }
    lo = s.pad_b;
    hi = min(s.offset + s.L - 1, s.len_b - 1);
    if (s.window > 0) lo = max(lo, s.offset - s.window + 1);
}

// Whether some query position l in [0, L) sees no key row at all.  The quantized path fills
// masked scores with finfo.min instead of dropping them (KVCache.swift:2396-2447), so such a
// row attends uniformly over ALL presented keys and no key tile may be skipped for it.
__device__ __forceinline__ bool sym_mask_some_row_empty(const SymMask &s) {
    if (s.mode == KVHIP_MASK_CAUSAL) return s.T - s.L < 0;
    // per position l the kept rows are [max(pad, offset + l - window + 1), min(offset + l, len - 1)]:
    // the width is concave in l, so it is smallest at one of the two ends
    for (int e = 0; e < 2; ++e) {
        const int l = e ? s.L - 1 : 0;
        int lo = s.pad_b;
        const int hi = min(s.offset + l, min(s.len_b, s.T) - 1);
        if (s.window > 0) lo = max(lo, s.offset + l - s.window + 1);
        if (lo > hi) return true;
    }
    return false;
}

// Inclusive range of key rows EVERY query position l in [0, L) sees (empty if lo > hi).
__device__ __forceinline__ void sym_mask_full_range(const SymMask &s, int &lo, int &hi) {
    if (s.mode == KVHIP_MASK_CAUSAL) {
        lo = 0;
        hi = s.T - s.L;
        return;
    }
    lo = s.pad_b;
    hi = min(s.offset, s.len_b - 1);
    if (s.window > 0) lo = max(lo, s.offset + s.L - s.window);
}

// ---- which batch row a workgroup row takes, for ragged batches ------------------------------------
// Workgroups are started in id order, one per CU and then a second one per CU, so rows v and v + B/2 of a
// launch of 512 workgroups share CUs.  Taking the batch rows in order of their visible length -- the first
// half of the workgroup rows in descending order, the second half in ascending order -- pairs the longest
// row with the shortest on the same CUs, the second longest with the second shortest, and so on, instead of
// whatever the batch order happens to pair.  Every workgroup computes the same permutation (one lane
// per batch row, B <= 64); partial results are still indexed by the batch row itself, so nothing
// downstream changes.
__device__ __forceinline__ int balanced_row(const MaskDev &m, int B, int L, int T, int tiles_total, int v) {
    const int lane = threadIdx.x & 63;
    int tiles = -1;
    if (lane < B) {
        const SymMask s = sym_mask_init(m, lane, L, T);
        int vis_lo, vis_hi;
        sym_mask_row_range(s, vis_lo, vis_hi);
        int t_lo = max(0, vis_lo) >> 6, t_hi = min(tiles_total, (min(vis_hi, T - 1) >> 6) + 1);
        if (sym_mask_some_row_empty(s)) {
            t_lo = 0;
            t_hi = tiles_total;
        }
        tiles = max(t_hi - t_lo, 0);
    }
    int rank = 0;  // rows that come before this lane's: more tiles, or as many and a lower index
    for (int j = 0; j < B; ++j) {
        const int tj = __shfl(tiles, j);
        rank += (tj > tiles || (tj == tiles && j < lane)) ? 1 : 0;
    }
    const int h = (B + 1) / 2;
    const int want = v < h ? v : B - 1 - (v - h);
    const unsigned long long hit = __ballot(lane < B && rank == want);
    return hit ? __ffsll(hit) - 1 : v;
}

}  // namespace kvhip
