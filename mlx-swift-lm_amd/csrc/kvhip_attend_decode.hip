// Split-sequence decode attention on the matrix cores (gfx950).
//
// One workgroup (4 wavefronts) owns a contiguous span of physical slots of one
// (batch, kv-head) pair and leaves an unnormalised partial (max, sum, out[D]) per
// query row; a second small kernel merges the partials of all spans.  All query
// rows that share a kv head (r = Hq/Hkv heads times L new tokens, up to 16) are
// served from one pass over K and V, which are read from HBM exactly once.
//
// The contraction uses v_mfma_f32_4x4x4_16B_f16: sixteen independent 4x4x4 blocks
// per instruction.  With CBSZ=4 the A operand of ONE block (chosen by ABID) is
// broadcast to all sixteen, so the small operand (4 query rows / 4 probability
// rows) costs two registers while the large one (K, V) fills the B side:
//
//   QK^T  block b covers tokens 4b..4b+3: lane l supplies four head-dim elements
//         of token l's K row (B); the accumulator of lane l receives the scores of
//         token l for the 4 query rows.  The query operands of 16 successive steps
//         live in the 16 lane groups of one register pair; ABID picks the step.
//   PV    block b covers head-dim columns 4b..4b+3 (+64h): lane l supplies, for
//         column l, four consecutive tokens of the transposed V tile (B); the
//         probabilities of step s (tokens 4s..4s+3) sit in lane group s after a
//         4x4 transpose inside each quad of lanes and are broadcast with ABID = s.
//
// Packed codes become operands without a dequantize pass: a code masked in place
// is the fp16 subnormal code * 2^-24 (high nibbles: * 2^-20, compensated by
// operands pre-scaled by 1/16), which the matrix core multiplies exactly.  So
//   q . (scale*code + bias)            = scale * 2^24 * mfma(q, masked K words) + bias * sum(q)
//   sum_t p_t (scale_t*code_t + bias_t) = 2^24 * mfma(p*scale, masked V words) + sum_t p_t bias_t
#include <cstdlib>
#include <utility>
#include <vector>

#include "kvhip_mask.hpp"

// piece buffers of the full-precision decode kernel (at most the D / 32 pieces of one tile)
#ifndef KVHIP_DECODE_FP_NBUF
#define KVHIP_DECODE_FP_NBUF(D, RG) 2
#endif

namespace kvhip {

namespace {

typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef short s4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
union Op {  // one 4-element 16-bit operand
    h4 h;
    s4 s;
    uint32_t u[2];
};

constexpr int WAVES = 4;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float TWO24 = 16777216.0f;

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(std::integral_constant<int, i>) for i = 0..N-1, fully unrolled with compile-time i
template <int N, class F> __device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <int ABID> __device__ __forceinline__ f4 mfma444(const Op &a, const Op &b, f4 c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(a.h, b.h, c, 4, ABID, 0);
}
template <int ABID> __device__ __forceinline__ f4 mfma444_bf(const Op &a, const Op &b, f4 c) {
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(a.s, b.s, c, 4, ABID, 0);
}

// v_exp_f32 without the denormal-range fix-up (results below 2^-126 flush to zero)
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Wavefront reductions on the data-parallel-primitive path (no LDS round trips): two quad
// permutes and two row mirrors leave each row of 16 lanes reduced, two row broadcasts
// carry the rows into lane 63, which is read out as a wave-uniform scalar.
template <int CTRL, int ROWS>
__device__ __forceinline__ float dpp_take(float v) {  // v of the lane CTRL names; own v outside ROWS
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                 CTRL, ROWS, 0xF, false));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_take<0xB1, 0xF>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_take<0x4E, 0xF>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_take<0x141, 0xF>(v));  // row_half_mirror
    v = fmaxf(v, dpp_take<0x140, 0xF>(v));  // row_mirror
    v = fmaxf(v, dpp_take<0x142, 0xA>(v));  // row_bcast15 into rows 1 and 3
    v = fmaxf(v, dpp_take<0x143, 0xC>(v));  // row_bcast31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_take<0xB1, 0xF>(v);
    v += dpp_take<0x4E, 0xF>(v);
    v += dpp_take<0x141, 0xF>(v);
    v += dpp_take<0x140, 0xF>(v);
    // the broadcast steps must add only into the rows they target
    const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));
    v += r1;
    const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));
    v += r2;
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float uniform(float v) {  // v is the same in every lane
    return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}
__device__ __forceinline__ uint16_t f2h_bits(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
__device__ __forceinline__ uint32_t pack_h2(float lo, float hi) { return pk_h2(lo, hi); }

// value held by lane (l ^ 1) / (l ^ 2) of the same quad
__device__ __forceinline__ uint32_t quad_xor1(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
}
__device__ __forceinline__ uint32_t quad_xor2(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
}
// 4x4 transpose inside each quad: before, lane c holds x[i]; after, lane i holds in
// x[k] what lane k held in x[i].
__device__ __forceinline__ void quad_transpose(uint32_t x[4], int lane) {
    const bool b0 = lane & 1, b1 = lane & 2;
    {
        const uint32_t s01 = b0 ? x[0] : x[1], s23 = b0 ? x[2] : x[3];
        const uint32_t r01 = quad_xor1(s01), r23 = quad_xor1(s23);
        x[0] = b0 ? r01 : x[0];
        x[1] = b0 ? x[1] : r01;
        x[2] = b0 ? r23 : x[2];
        x[3] = b0 ? x[3] : r23;
    }
    {
        const uint32_t s02 = b1 ? x[0] : x[2], s13 = b1 ? x[1] : x[3];
        const uint32_t r02 = quad_xor2(s02), r13 = quad_xor2(s13);
        x[0] = b1 ? r02 : x[0];
        x[2] = b1 ? x[2] : r02;
        x[1] = b1 ? r13 : x[1];
        x[3] = b1 ? x[3] : r13;
    }
}

// load N consecutive dwords with the widest vector accesses
// (from device memory: a `gptr`, so that the loads are GLOBAL rather than FLAT ones)
template <int N> __device__ __forceinline__ void load_words(uint32_t *dst, gptr p) {
    if constexpr (N % 4 == 0) {
#pragma unroll
        for (int i = 0; i < N / 4; ++i) {
            const kv_u4 v = ld_global<kv_u4>(p, i);
            dst[4 * i] = v.x; dst[4 * i + 1] = v.y; dst[4 * i + 2] = v.z; dst[4 * i + 3] = v.w;
        }
    } else if constexpr (N % 2 == 0) {
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
            const kv_u2 v = ld_global<kv_u2>(p, i);
            dst[2 * i] = v.x; dst[2 * i + 1] = v.y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) dst[i] = ld_global<uint32_t>(p, i);
    }
}

// ---- operand geometry --------------------------------------------------------------
// A "step" contracts 4 elements; one packed 32-bit word yields WSTEPS steps.
//   4 bit: 8 codes -> 2 steps taking nibbles (0,4,1,5) and (2,6,3,7); the last two
//          of each are high nibbles (value x16)
//   8 bit: 4 codes -> 1 step taking bytes (0,2,1,3)
template <int BITS> struct Geo;
template <> struct Geo<4> {
    static constexpr int WSTEPS = 2, EPW = 8;
    static __device__ __forceinline__ constexpr int elem(int h, int k) { return 2 * h + (k >> 1) + 4 * (k & 1); }
    static __device__ __forceinline__ constexpr bool hi(int k) { return k >= 2; }
    static __device__ __forceinline__ void unpack(uint32_t w, Op *o) {
        const uint32_t w8 = w >> 8;
        o[0].u[0] = w & 0x000f000fu;
        o[0].u[1] = w & 0x00f000f0u;
        o[1].u[0] = w8 & 0x000f000fu;
        o[1].u[1] = w8 & 0x00f000f0u;
    }
};
template <> struct Geo<8> {
    static constexpr int WSTEPS = 1, EPW = 4;
    static __device__ __forceinline__ constexpr int elem(int, int k) { return (k >> 1) + 2 * (k & 1); }
    static __device__ __forceinline__ constexpr bool hi(int) { return false; }
    static __device__ __forceinline__ void unpack(uint32_t w, Op *o) {
        o[0].u[0] = w & 0x00ff00ffu;
        o[0].u[1] = (w >> 8) & 0x00ff00ffu;
    }
};

// One tile (64 slots) of raw operand data in registers; lane l owns token l of the tile
// for K and head-dim column l (+64h) for V.
template <int BITS, int D, int G> struct TileRegs {
    static constexpr int KW = D * BITS / 32;   // dwords of one K row
    static constexpr int VW = 64 * BITS / 32;  // dwords of one V tile row
    uint32_t k[KW];
    uint32_t v[D / 64][VW];
    float ks[G], kb[G], vs[G], vb[G];
    int row;    // presented row of this lane's token, -1 if none
    bool edge;  // wave-uniform: some token of the tile is dead or masked for some query row
};

// RG = groups of 4 query rows handled per pass (R <= 4 RG).  MM selects the mask code:
// 0 none (the tile loop is branch free), 1 index-only masks (causal / window, per-batch
// bounds preloaded: no memory access in the loop), 2 array masks (loads in the loop, which
// force conservative waits on the prefetch).  Slots map to presented rows one to one: only
// RotatingKVCache remaps slots, and it is never quantized.
// NW = wavefronts per workgroup: 4 (two workgroups per CU), or 8 when that lets one
// workgroup take the whole sequence of its (batch, kv-head) pair -- then the output rows are
// normalised and written here and no partial goes through memory.
template <int BITS, int D, int GS, int DT, int RG, int MM, int NW>
__global__ void __launch_bounds__(NW * 64, NW == 4 ? 2 : 1)
decode_kernel(AttendArgs a, int tiles_total, int tiles_per_wg, int nsplit) {
    using GEO = Geo<BITS>;
    constexpr int G = D / GS;      // quantization groups per row (1, 2 or 4)
    constexpr int NH = D / 64;     // 64-column halves of the output
    constexpr int NQA = D / 64;    // query operand register pairs (16 steps of 4 elements each)
    constexpr int RR = 4 * RG;     // query rows carried
    // Group size 32: the 64 columns a PV instruction covers lie in two groups, and the probability
    // operand (which carries the V scale) is the same for every lane.  Each V step is therefore
    // issued twice, once with either group's operand, into two accumulators; lanes 0-31 keep the
    // first, lanes 32-63 the second.
    constexpr bool HALF = GS < 64;
    constexpr int NO2 = HALF ? D / 64 : 1;  // second accumulators (one dummy when unused)
    using T = TileRegs<BITS, D, G>;
    const Store &st = a.st;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform
    const int blk = lane >> 2, qi = lane & 3;  // lane group (MFMA block) and position in it
    int bh = blockIdx.y;
    const int split = blockIdx.x;
    int b = bh / a.Hkv;
    const int hk = bh - b * a.Hkv;
    if constexpr (MM == 1) {
        // a ragged batch whose rows divide their own ranges over the same number of spans: long and short
        // rows are paired on the CUs (balanced_row); partials stay indexed by the batch row itself
        if (tiles_per_wg == 0 && a.B <= 64 && a.B > 2) {
            b = __builtin_amdgcn_readfirstlane(balanced_row(a.mask, a.B, a.L, a.T, tiles_total, b));
            bh = b * a.Hkv + hk;
        }
    }
    const int r = a.Hq / a.Hkv;
    const int R = r * a.L;

    __shared__ float cbuf[NW][RR][D + 2];

    // ---- query operands: lane (blk, qi) holds row qi's 4 elements of step 16 x + blk ----
    // qsum[rg][g][i] = sum over group g of the (rounded, fp16-held) query row 4 rg + i, for
    // the bias term; built from the same registers: the 16 steps of one operand pair lie in
    // one group (group sizes of 64 and more; with 32 the lane groups 0-7 and 8-15 feed two sums), so a lane sums its 4 elements, the 16
    // lane groups are added up by shuffles and the four rows are read out of their quad.
    // (Built by a lambda that the main loop calls after it has requested its first tile, so the
    // first K/V loads are in flight while the queries are fetched and reduced.)
    Op qa[RG][NQA];
    float qsum[RG][G][4];
    auto load_queries = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
        const int i = 4 * rg + qi;
        // rows past R read row 0 (in bounds) and count as zero: no branch around the loads, which
        // are then all in flight together instead of one after the other
        const bool ok = i < R;
        const int rep = ok ? i / a.L : 0, l = ok ? i - rep * a.L : 0;
        const size_t qoff = ((size_t)(b * a.Hq + hk * r + rep) * a.L + l) * D;
        float raw[NQA][4];
#pragma unroll
        for (int x = 0; x < NQA; ++x) {
            const int step = 16 * x + blk;
            const int w = step / GEO::WSTEPS, h = step % GEO::WSTEPS;
#pragma unroll
            for (int k = 0; k < 4; ++k) raw[x][k] = Elem<DT>::load(a.q, qoff + w * GEO::EPW + GEO::elem(h, k));
        }
        float part[G];
#pragma unroll
        for (int g = 0; g < G; ++g) part[g] = 0.f;
#pragma unroll
        for (int x = 0; x < NQA; ++x) {
            float qv[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float v = ok ? (float)(_Float16)round_dt<DT>(raw[x][k] * a.scale) : 0.f;
                if constexpr (HALF) {  // steps 16 x + blk: lane groups 0-7 are one group of 32, 8-15 the next
                    part[2 * x] += blk < 8 ? v : 0.f;
                    part[2 * x + 1] += blk < 8 ? 0.f : v;
                } else {
                    part[(64 * x) / GS] += v;
                }
                qv[k] = GEO::hi(k) ? v * 0.0625f : v;
            }
            qa[rg][x].u[0] = pack_h2(qv[0], qv[1]);
            qa[rg][x].u[1] = pack_h2(qv[2], qv[3]);
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float v = part[g];
            for (int off = 4; off < 64; off <<= 1) v += __shfl_xor(v, off);  // over the 16 lane groups
#pragma unroll
            for (int ii = 0; ii < 4; ++ii)  // wave-uniform: keep it in a scalar register
                qsum[rg][g][ii] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), ii));
        }
    }
    };

    // ---- running state ---------------------------------------------------------------
    // m_use = m_run, or 0 while m_run is still -inf, so exp2((s - m_use) log2 e) needs no guard
    float m_run[RG][4], m_use[RG][4], l_part[RG][4], bacc[RG][G][4];
    f4 oacc[RG][NH];
    f4 oacc2[RG][NO2];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
        for (int h = 0; h < NO2; ++h) oacc2[rg][h] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 4; ++i) { m_run[rg][i] = -INFINITY; m_use[rg][i] = 0.f; l_part[rg][i] = 0.f; }
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) bacc[rg][g][i] = 0.f;
#pragma unroll
        for (int h = 0; h < NH; ++h) oacc[rg][h] = f4{0.f, 0.f, 0.f, 0.f};
    }

    const float fill = finfo_min_dt(DT);
    const SymMask sym = sym_mask_init(a.mask, b, a.L, a.T);
    int tile_begin = split * tiles_per_wg;
    int tile_end = min(tiles_total, tile_begin + tiles_per_wg);
    if constexpr (MM == 1) {
        // length-aware partition: an index-only mask bounds the rows this (batch) can see
        // (left padding, lengths, causal/window reach); spans of equal size start at the first
        // visible tile, so a ragged batch gets workgroups in proportion to each length
        int vis_lo, vis_hi;
        sym_mask_row_range(sym, vis_lo, vis_hi);
        int t_lo = max(0, vis_lo) >> 6, t_hi = min(tiles_total, (min(vis_hi, a.T - 1) >> 6) + 1);
        if (sym_mask_some_row_empty(sym)) {  // a fully masked row averages over every key
            t_lo = 0;
            t_hi = tiles_total;
        }
        // tiles_per_wg == 0: divide this batch row's own visible range over the spans
        const int per = tiles_per_wg > 0 ? tiles_per_wg
                                         : (max(t_hi - t_lo, 1) + nsplit * NW - 1) / (nsplit * NW) * NW;
        tile_begin = t_lo + split * per;  // spans past t_hi are empty
        tile_end = min(t_hi, tile_begin + per);
    }
    int mrow_l[RG][4];  // query position l of each carried row
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
        for (int i = 0; i < 4; ++i) mrow_l[rg][i] = (4 * rg + i) % a.L;
    // tokens whose V code sits in a high nibble carry 1/16 on the probability side
    const float vfac = (BITS == 4 && (lane & 2)) ? 0.0625f : 1.0f;

    constexpr int VROW = T::VW * 4;  // bytes of one V tile row

    // This wavefront takes tiles tile0, tile0 + NW, ...: always the same tile of
    // successive pages (4 tiles each), so its four plane pointers advance by NW / 4 page
    // cell strides.
    const int tile0 = tile_begin + wave;
    const int my_tiles = tile0 < tile_end ? (tile_end - tile0 + NW - 1) / NW : 0;
    constexpr int PSTEP = NW / 4;  // pages per step
    // pages are found through the page table: one scalar load per plane pair and page; the
    // offsets of this (b, kv-head)'s cell and of the tile inside it are the same in every page
    const int tip = tile0 & 3;  // 4 tiles per page
    int page_k = my_tiles > 0 ? tile0 >> 2 : 0, page_v = page_k;
    const size_t k_off = (size_t)bh * st.k_cell + (size_t)tip * TILE * st.k_row;
    const size_t v_off = (size_t)bh * st.v_cell + (size_t)tip * D * VROW;
    const size_t ksb_off = (size_t)bh * st.ksb_cell + (size_t)tip * TILE * st.ksb_row;
    const size_t vsb_off = (size_t)bh * st.vsb_cell + (size_t)tip * TILE * st.vsb_row;
    gptr kp = as_global(st.pt[page_k].k) + k_off;
    gptr vp = as_global(st.pt[page_k].v) + v_off;
    gptr ksp = as_global(st.pt[page_k].ksb) + ksb_off;
    gptr vsp = as_global(st.pt[page_k].vsb) + vsb_off;
    const uint32_t k_lane = lane * st.k_row, v_lane = lane * VROW;
    const uint32_t ksb_lane = lane * st.ksb_row, vsb_lane = lane * st.vsb_row;
    int slot_next = tile0 * TILE + lane;  // slot of this lane's token in the tile loaded next
    int base_next = tile0 * TILE;         // its first slot (wave-uniform)
    // rows every query row keeps: tiles inside [full_lo, full_hi] need no mask or bound test
    int full_lo = 0, full_hi = a.T - 1;
    if constexpr (MM == 1) {
        sym_mask_full_range(sym, full_lo, full_hi);
        full_hi = min(full_hi, a.T - 1);
    }

    // ---- the step's new row, when it is still to be written (unmasked single-token decode) -----
    // Slot T - 1 lies in the last tile, which exactly one wavefront of one workgroup reads (spans
    // are equal and cover every tile): that wavefront quantizes the row into the cache before it
    // requests any tile, with the arithmetic of the append kernel, so its own later loads of the
    // tile see it.  The V code goes into its column's packed word read-modify-write.
    if constexpr (MM == 0 && RG == 1) {
        if (a.new_k != nullptr) {  // wave-uniform
            const int slot = a.new_slot, tl = slot >> 6;
            if (tl >= tile_begin && tl < tile_end && ((tl - tile_begin) % NW) == wave) {
                const char *krow = static_cast<const char *>(a.new_k) + (size_t)bh * D * 2;
                const char *vrow = static_cast<const char *>(a.new_v) + (size_t)bh * D * 2;
                quantize_row_wave_from<DT, BITS>([&](int d) { return Elem<DT>::load(krow, d); }, D, GS, lane,
                                                 reinterpret_cast<uint32_t *>(const_cast<char *>(k_row_ptr(st, bh, slot))),
                                                 [](int, uint32_t) {}, const_cast<char *>(ksb_row_ptr(st, bh, slot)), nullptr, nullptr);
                char *vcell = const_cast<char *>(v_cell_ptr(st, bh, slot));
                const int bp = v_bitpos<BITS>(slot & (TILE - 1));
                quantize_row_wave_from<DT, BITS>(
                    [&](int d) { return Elem<DT>::load(vrow, d); }, D, GS, lane, nullptr,
                    [&](int d, uint32_t code) {
                        uint32_t *p = reinterpret_cast<uint32_t *>(vcell + v_row_off(st, slot, d)) + (bp >> 5);
                        *p = (*p & ~(((1u << BITS) - 1u) << (bp & 31))) | (code << (bp & 31));
                    },
                    const_cast<char *>(vsb_row_ptr(st, bh, slot)), nullptr, nullptr);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            }
        }
    }

    // The K half (codes, scales, row bookkeeping) and the V half of tile number k_loaded /
    // v_loaded of this wavefront (clamped to its last tile, so loads past the end stay
    // unconditional and in bounds).
    int k_loaded = 0, v_loaded = 0;
    auto load_k = [&](T &t) {
        load_words<T::KW>(t.k, kp + k_lane);
        uint32_t kraw[G];  // (scale, bias) pairs of a 16-bit dtype
        load_words<G>(kraw, ksp + ksb_lane);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (DT == 0) {
                t.ks[g] = (float)__builtin_bit_cast(_Float16, (uint16_t)kraw[g]);
                t.kb[g] = (float)__builtin_bit_cast(_Float16, (uint16_t)(kraw[g] >> 16));
            } else {
                t.ks[g] = __uint_as_float(kraw[g] << 16);
                t.kb[g] = __uint_as_float(kraw[g] & 0xffff0000u);
            }
        }
        t.row = slot_next < a.T ? slot_next : -1;
        t.edge = base_next < full_lo || base_next + (TILE - 1) > full_hi;
        ++k_loaded;
        if (k_loaded < my_tiles) {  // wave-uniform: step to the same tile of the next page
            page_k += PSTEP;
            kp = as_global(st.pt[page_k].k) + k_off;
            ksp = as_global(st.pt[page_k].ksb) + ksb_off;
            slot_next += PAGE * PSTEP;
            base_next += PAGE * PSTEP;
        }
    };
    auto load_v = [&](T &t) {
#pragma unroll
        for (int h = 0; h < NH; ++h) load_words<T::VW>(t.v[h], vp + v_lane + (size_t)h * 64 * VROW);
        uint32_t vraw[G];
        load_words<G>(vraw, vsp + vsb_lane);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (DT == 0) {
                t.vs[g] = (float)__builtin_bit_cast(_Float16, (uint16_t)vraw[g]);
                t.vb[g] = (float)__builtin_bit_cast(_Float16, (uint16_t)(vraw[g] >> 16));
            } else {
                t.vs[g] = __uint_as_float(vraw[g] << 16);
                t.vb[g] = __uint_as_float(vraw[g] & 0xffff0000u);
            }
        }
        ++v_loaded;
        if (v_loaded < my_tiles) {
            page_v += PSTEP;
            vp = as_global(st.pt[page_v].v) + v_off;
            vsp = as_global(st.pt[page_v].vsb) + vsb_off;
        }
    };
    auto load_tile = [&](T &t) {
        load_k(t);
        load_v(t);
    };

    Op pa[RG][G];  // probabilities of the tile in flight, as PV operands
    auto compute_qk_softmax = [&](const T &t) {
        const bool live = t.row >= 0;
        // ---- QK^T: scores of token `lane` for every query row ---------------------------
        f4 sacc[RG][G];
#pragma unroll
        for (int rg = 0; rg < RG; ++rg)
#pragma unroll
            for (int g = 0; g < G; ++g) sacc[rg][g] = f4{0.f, 0.f, 0.f, 0.f};
        static_for<T::KW>([&](auto W) {
            constexpr int w = decltype(W)::value;
            constexpr int g = (w * GEO::EPW) / GS;
            Op o[GEO::WSTEPS];
            GEO::unpack(t.k[w], o);
            static_for<GEO::WSTEPS>([&](auto H) {
                constexpr int h = decltype(H)::value;
                constexpr int step = w * GEO::WSTEPS + h;
#pragma unroll
                for (int rg = 0; rg < RG; ++rg)
                    sacc[rg][g] = mfma444<step % 16>(qa[rg][step / 16], o[h], sacc[rg][g]);
            });
        });

        // ---- online softmax per row group; probabilities become PV A operands ------------
        // Interior tiles (every token live and visible to every query row: the common case,
        // decided per wavefront when the tile was loaded) skip all mask and bound tests.
        float ks24[G], vsf[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            ks24[g] = t.ks[g] * TWO24;
            vsf[g] = t.vs[g] * vfac;
        }
        auto softmax_rg = [&](auto RGC) {
            constexpr int rg = decltype(RGC)::value;
            float sc[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float s_ = t.kb[0] * qsum[rg][0][i];
#pragma unroll
                for (int g = 1; g < G; ++g) s_ = __builtin_fmaf(t.kb[g], qsum[rg][g][i], s_);
#pragma unroll
                for (int g = 0; g < G; ++g) s_ = __builtin_fmaf(ks24[g], sacc[rg][g][i], s_);
                sc[i] = round_dt<DT>(s_);
            }
            if (MM == 2 || t.edge) {  // wave-uniform
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float s_ = sc[i];
                    [[maybe_unused]] const int row_i = 4 * rg + i;
                    if constexpr (MM == 1) {
                        if (!sym_mask_keep(sym, mrow_l[rg][i], t.row)) s_ = fill;
                    } else if constexpr (MM == 2) {
                        if (live && row_i < R) {
                            const int rep = row_i / a.L, l = row_i - rep * a.L;
                            float add;
                            const bool keep = mask_keep(a.mask, b, hk * r + rep, l, t.row, a.L, a.T, add);
                            if (!keep) s_ = fill;
                            else if (a.mask.dtype != KVHIP_BOOL) s_ = round_dt<DT>(s_ + add);
                        }
                    }
                    sc[i] = live ? s_ : -INFINITY;
                }
            }
            // raise the running maximum only when this tile exceeds it (rare after the first
            // few tiles; the empty asm keeps the reductions inside the branch)
            bool need = false;
#pragma unroll
            for (int i = 0; i < 4; ++i) need = need || (sc[i] > m_run[rg][i]);
            if (__any(need)) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float x_ = sc[i];
                    asm volatile("" : "+v"(x_));
                    // wave-uniform values, kept in scalar registers
                    const float mn = uniform(fmaxf(m_run[rg][i], wave_max(x_)));
                    const float alpha = (mn == -INFINITY) ? 1.f : fast_exp2((m_run[rg][i] - mn) * LOG2E);
                    m_run[rg][i] = mn;
                    m_use[rg][i] = uniform((mn == -INFINITY) ? 0.f : mn);
                    l_part[rg][i] *= alpha;
#pragma unroll
                    for (int g = 0; g < G; ++g) bacc[rg][g][i] *= alpha;
#pragma unroll
                    for (int h = 0; h < NH; ++h) oacc[rg][h][i] *= alpha;
                    if constexpr (HALF) {
#pragma unroll
                        for (int h = 0; h < NH; ++h) oacc2[rg][h][i] *= alpha;
                    }
                }
            }
            constexpr int GP = (G + 1) / 2;  // groups travel through the transpose two to a register
            uint32_t x[GP][4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // exp2(-inf) = 0 covers dead lanes; m_use is finite even before any live token
                const float p = fast_exp2((sc[i] - m_use[rg][i]) * LOG2E);
                l_part[rg][i] += p;
                float pv[2 * GP];
                pv[2 * GP - 1] = 0.f;
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    bacc[rg][g][i] = __builtin_fmaf(p, t.vb[g], bacc[rg][g][i]);
                    pv[g] = p * vsf[g];
                }
#pragma unroll
                for (int j = 0; j < GP; ++j) x[j][i] = pack_h2(pv[2 * j], pv[2 * j + 1]);
            }
            // lane (blk, i) now gets, in x[j][k], row i's value for token 4 blk + k
#pragma unroll
            for (int j = 0; j < GP; ++j) {
                quad_transpose(x[j], lane);
                pa[rg][2 * j].u[0] = __builtin_amdgcn_perm(x[j][1], x[j][0], 0x05040100u);
                pa[rg][2 * j].u[1] = __builtin_amdgcn_perm(x[j][3], x[j][2], 0x05040100u);
                if (2 * j + 1 < G) {
                    pa[rg][2 * j + 1].u[0] = __builtin_amdgcn_perm(x[j][1], x[j][0], 0x07060302u);
                    pa[rg][2 * j + 1].u[1] = __builtin_amdgcn_perm(x[j][3], x[j][2], 0x07060302u);
                }
            }
        };
        static_for<RG>([&](auto RGC) { softmax_rg(RGC); });
    };

    // ---- out += P . V: lane supplies column lane (+64 h), step s = tokens 4s..4s+3 ----------
    auto compute_pv = [&](const T &t) {
        static_for<NH>([&](auto HH) {
            constexpr int h = decltype(HH)::value;
            constexpr int g = HALF ? 2 * h : (64 * h) / GS;
            static_for<T::VW>([&](auto W) {
                constexpr int w = decltype(W)::value;
                Op o[GEO::WSTEPS];
                GEO::unpack(t.v[h][w], o);
                static_for<GEO::WSTEPS>([&](auto S2) {
                    constexpr int s = w * GEO::WSTEPS + decltype(S2)::value;
#pragma unroll
                    for (int rg = 0; rg < RG; ++rg) {
                        oacc[rg][h] = mfma444<s>(pa[rg][g], o[decltype(S2)::value], oacc[rg][h]);
                        if constexpr (HALF)
                            oacc2[rg][h] = mfma444<s>(pa[rg][g + 1], o[decltype(S2)::value], oacc2[rg][h]);
                    }
                });
            });
        });
    };

    auto compute_tile = [&](const T &t) {
        compute_qk_softmax(t);
        compute_pv(t);
    };

    // ---- main loop.  Variants whose tile fits twice in the register file keep one whole
    // tile of loads in flight ahead of the arithmetic.  The others run one buffer with the
    // halves skewed: V of a tile is requested before its QK^T and softmax, K of the next
    // tile before its PV, so each half has the other half's arithmetic to arrive in.
    constexpr bool PREFETCH = (RG == 1 && !(BITS == 8 && D >= 128)) || (BITS == 4 && D <= 128 && (RG == 2 || D == 64));
    if (my_tiles > 0) {
        if constexpr (PREFETCH) {
            T bufA, bufB;
            load_tile(bufA);
            load_queries();
            for (int done = 0;;) {
                load_tile(bufB);
                compute_tile(bufA);
                if (++done == my_tiles) break;
                load_tile(bufA);
                compute_tile(bufB);
                if (++done == my_tiles) break;
            }
        } else {
            T buf;
            load_k(buf);
            load_queries();
            for (int done = 0; done < my_tiles; ++done) {
                load_v(buf);
                compute_qk_softmax(buf);
                load_k(buf);
                compute_pv(buf);
            }
        }
    }

    // ---- wavefront partial -> LDS ---------------------------------------------------
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            l_part[rg][i] = wave_sum(l_part[rg][i]);
#pragma unroll
            for (int g = 0; g < G; ++g) bacc[rg][g][i] = wave_sum(bacc[rg][g][i]);
        }
#pragma unroll
        for (int h = 0; h < NH; ++h) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float o_ = oacc[rg][h][i], b_ = bacc[rg][HALF ? 2 * h : (64 * h) / GS][i];
                if constexpr (HALF) {
                    if (lane >= 32) {
                        o_ = oacc2[rg][h][i];
                        b_ = bacc[rg][2 * h + 1][i];
                    }
                }
                cbuf[wave][4 * rg + i][64 * h + lane] = o_ * TWO24 + b_;
            }
        }
        if (lane < 4) {
            cbuf[wave][4 * rg + lane][D] = m_run[rg][lane];
            cbuf[wave][4 * rg + lane][D + 1] = l_part[rg][lane];
        }
    }
    __syncthreads();
    // ---- merge the wavefronts; a single span writes the output rows, several leave partials
    if (nsplit == 1) {
        for (int idx = threadIdx.x; idx < R * D; idx += NW * 64) {
            const int i = idx / D, c = idx - i * D;
            float mx = -INFINITY;
#pragma unroll
            for (int w = 0; w < NW; ++w) mx = fmaxf(mx, cbuf[w][i][D]);
            float v = 0.f, l = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float mw = cbuf[w][i][D];
                const float wgt = (mw == -INFINITY) ? 0.f : fast_exp2((mw - mx) * LOG2E);
                v += wgt * cbuf[w][i][c];
                l += wgt * cbuf[w][i][D + 1];
            }
            const int rep = i / a.L, lq = i - rep * a.L;
            Elem<DT>::store(a.out, ((size_t)(b * a.Hq + hk * r + rep) * a.L + lq) * D + c, l > 0.f ? v / l : 0.f);
        }
        return;
    }
    float *part = a.workspace + ((size_t)bh * nsplit + split) * RR * (D + 2);
    for (int idx = threadIdx.x; idx < RR * (D + 2); idx += NW * 64) {
        const int i = idx / (D + 2), c = idx - i * (D + 2);
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) mx = fmaxf(mx, cbuf[w][i][D]);
        float v;
        if (c == D) {
            v = mx;
        } else {
            v = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float mw = cbuf[w][i][D];
                const float wgt = (mw == -INFINITY) ? 0.f : fast_exp2((mw - mx) * LOG2E);
                v += wgt * cbuf[w][i][c];
            }
        }
        part[idx] = v;
    }
}

// ---------------------------------------------------------------------------------
// Full-precision caches (KVCacheSimple, RotatingKVCache), fp16 or bf16.
//
// Same decomposition and the same 4x4x4 broadcast contraction as above, but a tile of
// 16-bit K and V is 4x larger than a 4-bit one, so it is streamed through two
// 32-register buffers in pieces of 64 elements per lane: a K piece is 64 head-dim
// elements of the lane's token, a V piece is the 64 tokens of the lane's column.
// The load of the next piece is issued as soon as a buffer has been consumed.
// bf16 keeps P as a (hi, lo) pair of bf16 values so the PV product carries 16 bits of
// probability; rows of a RotatingKVCache are found through the run table.
template <int D, int DT, int RG, int MM, bool IDENT>
__global__ void __launch_bounds__(WAVES * 64, 2)
decode_fp_kernel(AttendArgs a, int tiles_total, int tiles_per_wg, int nsplit) {
    constexpr bool BF = DT == 1;
    constexpr int NP = D / 64;   // pieces per K row and per V tile column set
    constexpr int RR = 4 * RG;
    constexpr int PW = 32;       // dwords per piece
    const Store &st = a.st;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int blk = lane >> 2, qi = lane & 3;
    const int bh = blockIdx.y, split = blockIdx.x;
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int r = a.Hq / a.Hkv;
    const int R = r * a.L;

    __shared__ float cbuf[WAVES][RR][D + 2];

    // query operands: lane (blk, qi) holds row qi's elements 4*(16 x + blk) .. +3, unscaled
    // (fetched by the main loop after it has requested its first two pieces)
    Op qa[RG][NP];
    auto load_queries = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
            const int i = 4 * rg + qi;
            const int rep = i / a.L, l = i - rep * a.L;
            const size_t qoff = ((size_t)(b * a.Hq + hk * r + rep) * a.L + l) * D;
#pragma unroll
            for (int x = 0; x < NP; ++x) {
                uint2 w = make_uint2(0, 0);
                if (i < R)
                    w = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(a.q) + qoff + 4 * (16 * x + blk));
                qa[rg][x].u[0] = w.x;
                qa[rg][x].u[1] = w.y;
            }
        }
    };

    float m_run[RG][4], l_part[RG][4];
    f4 oacc[RG][NP];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { m_run[rg][i] = -INFINITY; l_part[rg][i] = 0.f; }
#pragma unroll
        for (int h = 0; h < NP; ++h) oacc[rg][h] = f4{0.f, 0.f, 0.f, 0.f};
    }

    const SymMask sym = sym_mask_init(a.mask, b, a.L, a.T);
    int mrow_l[RG][4];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
        for (int i = 0; i < 4; ++i) mrow_l[rg][i] = (4 * rg + i) % a.L;
    int tile_begin = split * tiles_per_wg;
    int tile_end = min(tiles_total, tile_begin + tiles_per_wg);
    if constexpr (MM == 1 && IDENT) {
        int vis_lo, vis_hi;
        sym_mask_row_range(sym, vis_lo, vis_hi);
        const int t_lo = max(0, vis_lo) >> 6, t_hi = min(tiles_total, (min(vis_hi, a.T - 1) >> 6) + 1);
        // tiles_per_wg == 0: divide this batch row's own visible range over the spans
        const int per = tiles_per_wg > 0 ? tiles_per_wg
                                         : (max(t_hi - t_lo, 1) + nsplit * WAVES - 1) / (nsplit * WAVES) * WAVES;
        tile_begin = t_lo + split * per;  // spans past t_hi are empty
        tile_end = min(t_hi, tile_begin + per);
    }
    const int tile0 = tile_begin + wave;
    const int my_tiles = tile0 < tile_end ? (tile_end - tile0 + WAVES - 1) / WAVES : 0;
    // ---- the step's new row, when it is still to be written (unmasked single-token decode) -----
    // Exactly one wavefront of one workgroup reads the tile of physical slot `new_slot` (spans are equal and
    // cover every tile): it copies the row into the page before it requests any tile, so its own later
    // loads of the tile see it.
    if constexpr (MM == 0) {
        if (a.new_k != nullptr) {  // wave-uniform
            const int slot = a.new_slot, tl = slot >> 6;
            if (tl >= tile_begin && tl < tile_end && ((tl - tile_begin) % WAVES) == wave) {
                const uint16_t *krow = static_cast<const uint16_t *>(a.new_k) + (size_t)bh * D;
                const uint16_t *vrow = static_cast<const uint16_t *>(a.new_v) + (size_t)bh * D;
                char *kc = const_cast<char *>(k_cell_ptr(st, bh, slot));
                char *vc = const_cast<char *>(v_cell_ptr(st, bh, slot));
                if (lane < D / 8)  // one 16-byte chunk of the K row per lane
                    *reinterpret_cast<uint4 *>(kc + kfp_off(st, slot, 8 * lane)) = *reinterpret_cast<const uint4 *>(krow + 8 * lane);
                for (int d = lane; d < D; d += 64)
                    *reinterpret_cast<uint16_t *>(vc + vfp_off(st, slot, d)) = vrow[d];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            }
        }
    }
    // a wavefront's tiles are a page apart: each is found through the page table (a scalar load)
    const int tip = tile0 & 3;
    int page_k = my_tiles > 0 ? tile0 >> 2 : 0, page_v = page_k;
    constexpr int VROW = TILE * 2;  // bytes of one V tile row
    const size_t k_off = (size_t)bh * st.k_cell + (size_t)tip * TILE * st.k_row;
    const size_t v_off = (size_t)bh * st.v_cell + (size_t)tip * D * VROW;
    // (plain pointers, hence FLAT loads, on purpose: as GLOBAL loads with a scalar base the short launches
    // of this kernel measured 0.4-1 us slower -- 19.1 against 18.7 us on a 4096-row ring at D = 256,
    // 10.4-11.2 against 9.1-10.1 us at 1024 rows of D = 128 -- and the long ones the same)
    const char *kp = st.pt[page_k].k + k_off;
    const char *vp = st.pt[page_k].v + v_off;
    // chunk-interleaved tiles: chunk j of the lane's token (K) or column (V) sits 16 * lane bytes into
    // a 1 KB (K) / 16 D byte (V) row of chunks, so every load below is contiguous across the wavefront
    const uint32_t k_lane = lane * 16, v_lane = lane * 16;
    int slot_cur = tile0 * TILE + lane;
    int k_loaded = 0, v_loaded = 0;  // tiles whose K / V pieces have been requested
    auto load_chunks = [&](uint32_t *buf, const char *p, size_t stride) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < PW / 4; ++j) {
            const uint4 v = *reinterpret_cast<const uint4 *>(p + (size_t)j * stride);
            buf[4 * j] = v.x; buf[4 * j + 1] = v.y; buf[4 * j + 2] = v.z; buf[4 * j + 3] = v.w;
        }
    };

    // piece x of the K row / V column set of the tile the respective pointer stands on;
    // after the last piece the pointer steps to this wavefront's next tile (clamped, so
    // the prefetch past the end stays unconditional and in bounds)
    auto load_k = [&](uint32_t *buf, int x) {
        load_chunks(buf, kp + k_lane + (size_t)x * (PW / 4) * (TILE * 16), TILE * 16);  // chunks 8x .. 8x+7 of the lane's token
        if (x == NP - 1) {
            ++k_loaded;
            if (k_loaded < my_tiles) kp = st.pt[++page_k].k + k_off;
        }
    };
    auto load_v = [&](uint32_t *buf, int x) {
        load_chunks(buf, vp + v_lane + (size_t)x * 64 * 16, (size_t)D * 16);  // the 8 token chunks of column 64x + lane
        if (x == NP - 1) {
            ++v_loaded;
            if (v_loaded < my_tiles) vp = st.pt[++page_v].v + v_off;
        }
    };

    // piece order per tile: K0 .. K(NP-1), V0 .. V(NP-1); piece n lives in buffer n % NBUF and piece
    // n + NBUF is requested as soon as piece n has been consumed.  Two buffers: four (32 KB per
    // wavefront in flight) measured slower on the short launches they were meant for (a 4096-row
    // sliding window at D = 256, one tile per wavefront: 17.4 us against 15.7 us).
    constexpr int NBUF = KVHIP_DECODE_FP_NBUF(D, RG);
    uint32_t bufs[NBUF][PW];
    auto buf_of = [&](int n) -> uint32_t * { return bufs[n % NBUF]; };
    // request piece n (counted from the start of a tile; past its end: of the next tile) into `buf`
    auto request = [&](uint32_t *buf, int n) __attribute__((always_inline)) {
        n %= 2 * NP;
        if (n < NP) load_k(buf, n);
        else load_v(buf, n - NP);
    };

    if (my_tiles > 0) {
        // (the queries first: loads complete in order, and a wait for queries requested after the
        // first pieces would be a wait for those pieces too -- in every iteration, the compiler
        // placing one wait for all ways into the loop)
        load_queries();
        static_for<NBUF>([&](auto N) { request(buf_of(decltype(N)::value), decltype(N)::value); });
        for (int done = 0; done < my_tiles; ++done) {
            int row;
            if (IDENT) row = slot_cur;
            else row = slot_cur < a.slots ? slot_to_row(a.runs, slot_cur) : -1;
            row = (row >= 0 && row < a.T) ? row : -1;
            const bool live = row >= 0;
            // ---- QK^T over the K pieces ---------------------------------------------
            f4 sacc[RG];
#pragma unroll
            for (int rg = 0; rg < RG; ++rg) sacc[rg] = f4{0.f, 0.f, 0.f, 0.f};
            static_for<NP>([&](auto X) {
                constexpr int x = decltype(X)::value;
                uint32_t *buf = buf_of(x);
                static_for<16>([&](auto S) {
                    constexpr int s = decltype(S)::value;
                    Op o;
                    o.u[0] = buf[2 * s];
                    o.u[1] = buf[2 * s + 1];
#pragma unroll
                    for (int rg = 0; rg < RG; ++rg)
                        sacc[rg] = BF ? mfma444_bf<s>(qa[rg][x], o, sacc[rg]) : mfma444<s>(qa[rg][x], o, sacc[rg]);
                });
                // the buffer is free: request the piece NBUF ahead in the order K.., V.., next tile's K..
                request(buf, x + NBUF);
            });
            // ---- online softmax ----------------------------------------------------------
            Op pa[RG], pl[RG];
#pragma unroll
            for (int rg = 0; rg < RG; ++rg) {
                float sc[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float s_ = sacc[rg][i] * a.scale;
                    [[maybe_unused]] const int row_i = 4 * rg + i;
                    if constexpr (MM == 1) {
                        if (!sym_mask_keep(sym, mrow_l[rg][i], row)) s_ = -INFINITY;
                    } else if constexpr (MM == 2) {
                        if (live && row_i < R) {
                            const int rep = row_i / a.L, l = row_i - rep * a.L;
                            float add;
                            const bool keep = mask_keep(a.mask, b, hk * r + rep, l, row, a.L, a.T, add);
                            s_ = keep ? s_ + add : -INFINITY;
                        }
                    }
                    sc[i] = live ? s_ : -INFINITY;
                }
                bool need = false;
#pragma unroll
                for (int i = 0; i < 4; ++i) need = need || (sc[i] > m_run[rg][i]);
                if (__any(need)) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float x_ = sc[i];
                        asm volatile("" : "+v"(x_));  // keeps the reduction inside the branch
                        const float mn = fmaxf(m_run[rg][i], wave_max(x_));
                        const float alpha = (mn == -INFINITY) ? 1.f : fast_exp2((m_run[rg][i] - mn) * LOG2E);
                        m_run[rg][i] = mn;
                        l_part[rg][i] *= alpha;
#pragma unroll
                        for (int h = 0; h < NP; ++h) oacc[rg][h][i] *= alpha;
                    }
                }
                uint32_t xx[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float p = (sc[i] == -INFINITY || m_run[rg][i] == -INFINITY) ? 0.f : fast_exp2((sc[i] - m_run[rg][i]) * LOG2E);
                    l_part[rg][i] += p;
                    if (BF) {
                        const uint32_t hi = Elem<1>::bits(p);
                        const float rest = p - __uint_as_float(hi << 16);
                        xx[i] = hi | ((uint32_t)Elem<1>::bits(rest) << 16);
                    } else {
                        xx[i] = (uint32_t)f2h_bits(p);
                    }
                }
                quad_transpose(xx, lane);
                pa[rg].u[0] = __builtin_amdgcn_perm(xx[1], xx[0], 0x05040100u);
                pa[rg].u[1] = __builtin_amdgcn_perm(xx[3], xx[2], 0x05040100u);
                if (BF) {
                    pl[rg].u[0] = __builtin_amdgcn_perm(xx[1], xx[0], 0x07060302u);
                    pl[rg].u[1] = __builtin_amdgcn_perm(xx[3], xx[2], 0x07060302u);
                }
            }
            // ---- out += P . V over the V pieces ---------------------------------------------
            static_for<NP>([&](auto X) {
                constexpr int x = decltype(X)::value;
                uint32_t *buf = buf_of(NP + x);
                static_for<16>([&](auto S) {
                    constexpr int s = decltype(S)::value;
                    Op o;
                    o.u[0] = buf[2 * s];
                    o.u[1] = buf[2 * s + 1];
#pragma unroll
                    for (int rg = 0; rg < RG; ++rg) {
                        if (BF) {
                            oacc[rg][x] = mfma444_bf<s>(pa[rg], o, oacc[rg][x]);
                            oacc[rg][x] = mfma444_bf<s>(pl[rg], o, oacc[rg][x]);
                        } else {
                            oacc[rg][x] = mfma444<s>(pa[rg], o, oacc[rg][x]);
                        }
                    }
                });
                request(buf, NP + x + NBUF);
            });
            slot_cur += PAGE;
        }
    }

#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
        for (int i = 0; i < 4; ++i) l_part[rg][i] = wave_sum(l_part[rg][i]);
#pragma unroll
        for (int h = 0; h < NP; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) cbuf[wave][4 * rg + i][64 * h + lane] = oacc[rg][h][i];
        if (lane < 4) {
            cbuf[wave][4 * rg + lane][D] = m_run[rg][lane];
            cbuf[wave][4 * rg + lane][D + 1] = l_part[rg][lane];
        }
    }
    __syncthreads();
    // a single span writes the output rows itself, several leave partials for the merge kernel
    if (nsplit == 1) {
        for (int idx = threadIdx.x; idx < R * D; idx += WAVES * 64) {
            const int i = idx / D, c = idx - i * D;
            float mx = -INFINITY;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, cbuf[w][i][D]);
            float v = 0.f, l = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const float mw = cbuf[w][i][D];
                const float wgt = (mw == -INFINITY) ? 0.f : fast_exp2((mw - mx) * LOG2E);
                v += wgt * cbuf[w][i][c];
                l += wgt * cbuf[w][i][D + 1];
            }
            const int rep = i / a.L, lq = i - rep * a.L;
            Elem<DT>::store(a.out, ((size_t)(b * a.Hq + hk * r + rep) * a.L + lq) * D + c, l > 0.f ? v / l : 0.f);
        }
        return;
    }
    float *part = a.workspace + ((size_t)bh * nsplit + split) * RR * (D + 2);
    for (int idx = threadIdx.x; idx < RR * (D + 2); idx += WAVES * 64) {
        const int i = idx / (D + 2), c = idx - i * (D + 2);
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, cbuf[w][i][D]);
        float v;
        if (c == D) {
            v = mx;
        } else {
            v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const float mw = cbuf[w][i][D];
                const float wgt = (mw == -INFINITY) ? 0.f : fast_exp2((mw - mx) * LOG2E);
                v += wgt * cbuf[w][i][c];
            }
        }
        part[idx] = v;
    }
}

// grid (R, BH), 256 threads: merge the span partials of one query row and write the output row.
// A launch with few rows and many spans (a single sequence: 8 pairs, 32 to 512 spans each) lasts as long as its
// chain of memory round trips, so everything is asked for at once: a thread is (column pair, span group) and
// requests its first eight partial pairs before anything else, then the (max, sum) of up to two spans; the weights
// are formed while the columns are in flight, go through LDS, and the span groups' sums meet there at the end.
template <int D, int DT>
__global__ void __launch_bounds__(256) combine_kernel(AttendArgs a, int nsplit, int rr) {
    constexpr int CP = D / 2;     // column pairs
    constexpr int NG = 256 / CP;  // span groups: 8 (D 64), 6, 5, 4 (D 128), 2 (D 256)
    constexpr int UN = 8;         // loads in flight per thread and round
    __shared__ float w_s[512];    // weight of each span for this row (nsplit <= 512)
    __shared__ float red_s[2][4];
    __shared__ kv_f2 acc_s[NG][CP];
    const int i = blockIdx.x, bh = blockIdx.y;
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int r = a.Hq / a.Hkv;
    const int rep = i / a.L, l = i - rep * a.L;
    const size_t sstride = (size_t)rr * (D + 2);
    const size_t first_slot = (size_t)bh * nsplit;
    // (rows of D + 2 floats, D even: every pair below is 8-byte aligned)
    const float *part = a.workspace + first_slot * sstride + (size_t)i * (D + 2);
    const int t = threadIdx.x;
    const int g = t / CP, cp = t - g * CP;
    const bool col = g < NG;
    auto pair_at = [&](int s, int c) { return *reinterpret_cast<const kv_f2 *>(part + (size_t)s * sstride + c); };
    kv_f2 v[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const int s = g + NG * u;
        v[u] = (col && s < nsplit) ? pair_at(s, 2 * cp) : kv_f2{0.f, 0.f};
    }
    kv_f2 ml[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) ml[u] = t + 256 * u < nsplit ? pair_at(t + 256 * u, D) : kv_f2{-INFINITY, 0.f};
    float mloc = wave_max(fmaxf(ml[0].x, ml[1].x));
    if ((t & 63) == 0) red_s[0][t >> 6] = mloc;
    __syncthreads();
    const float mx = fmaxf(fmaxf(red_s[0][0], red_s[0][1]), fmaxf(red_s[0][2], red_s[0][3]));
    float dloc = 0.f;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const float w = (ml[u].x == -INFINITY) ? 0.f : fast_exp2((ml[u].x - mx) * LOG2E);
        if (t + 256 * u < nsplit) w_s[t + 256 * u] = w;
        dloc += w * ml[u].y;
    }
    dloc = wave_sum(dloc);
    if ((t & 63) == 0) red_s[1][t >> 6] = dloc;
    __syncthreads();
    const float den = (red_s[1][0] + red_s[1][1]) + (red_s[1][2] + red_s[1][3]);
    kv_f2 num{0.f, 0.f};
#pragma unroll
    for (int u = 0; u < UN; ++u) {
        const int s = g + NG * u;
        if (col && s < nsplit) num += w_s[s] * v[u];
    }
    for (int s0 = g + NG * UN; col && s0 < nsplit; s0 += NG * UN) {  // more than 8 NG spans: further rounds
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int s = s0 + NG * u;
            v[u] = s < nsplit ? pair_at(s, 2 * cp) : kv_f2{0.f, 0.f};
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int s = s0 + NG * u;
            if (s < nsplit) num += w_s[s] * v[u];
        }
    }
    if (col) acc_s[g][cp] = num;
    __syncthreads();
    if (t < CP) {
        kv_f2 o = acc_s[0][t];
#pragma unroll
        for (int k = 1; k < NG; ++k) o += acc_s[k][t];
        const float o0 = den > 0.f ? o.x / den : 0.f, o1 = den > 0.f ? o.y / den : 0.f;
        uint32_t *dst = reinterpret_cast<uint32_t *>(static_cast<char *>(a.out) + (((size_t)(b * a.Hq + hk * r + rep) * a.L + l) * D + 2 * t) * 2);
        *dst = DT == 0 ? pk_h2(o0, o1) : pk_bf2(o0, o1);
    }
}

// The same merge for the prefill tiles' key-range parts: many query rows, at most 8 parts.  One wavefront per
// query row, four rows per workgroup; a lane takes four adjacent columns; no LDS and no barrier (the
// per-row workgroups above spend their time being launched: 22 us for 16 384 rows of 256 columns).  Decode
// launches keep the kernel above: with few rows and many parts it has the loads of a column in flight together
// (configs[3]'s ring decode, 2 rows of 16 parts: 29.1 us per step against 31.7 us with this one).
template <int D, int DT>
__global__ void __launch_bounds__(256) combine_rows_kernel(AttendArgs a, int nsplit, int rr) {
    const int lane = threadIdx.x & 63;
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6), bh = blockIdx.y;
    const int r = a.Hq / a.Hkv;
    if (i >= r * a.L) return;  // (rr, the rows a part holds, may exceed the query rows there are)
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int rep = i / a.L, l = i - rep * a.L;
    const size_t sstride = (size_t)rr * (D + 2);
    const float *part = a.workspace + (size_t)bh * nsplit * sstride + (size_t)i * (D + 2);
    constexpr int MAXP = 8;
    float m[MAXP], w[MAXP];
    float mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < MAXP; ++s) {
        m[s] = s < nsplit ? part[s * sstride + D] : -INFINITY;
        mx = fmaxf(mx, m[s]);
    }
    float den = 0.f;
#pragma unroll
    for (int s = 0; s < MAXP; ++s) {
        w[s] = (m[s] == -INFINITY) ? 0.f : fast_exp2((m[s] - mx) * LOG2E);
        if (s < nsplit) den += w[s] * part[s * sstride + D + 1];
    }
    if (lane >= D / 4) return;
    float num[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < MAXP; ++s)
        if (s < nsplit) {
            // (a row of partials is 8-byte aligned: D + 2 floats)
            const float2 p0 = *reinterpret_cast<const float2 *>(part + s * sstride + 4 * lane);
            const float2 p1 = *reinterpret_cast<const float2 *>(part + s * sstride + 4 * lane + 2);
            num[0] += w[s] * p0.x;
            num[1] += w[s] * p0.y;
            num[2] += w[s] * p1.x;
            num[3] += w[s] * p1.y;
        }
    const size_t ooff = ((size_t)(b * a.Hq + hk * r + rep) * a.L + l) * D + 4 * lane;
#pragma unroll
    for (int c = 0; c < 4; ++c) Elem<DT>::store(a.out, ooff + c, den > 0.f ? num[c] / den : 0.f);
}

struct Plan {
    int tiles_total, tiles_per_wg, nsplit, rg, nw;
};

// Quantized shapes that run on the 16-row kernel at every row count: head size 96 (a row and a half of the 4-row
// kernel's 64-column halves), keys of 192 with values of 128, and 2-, 3-, 5- and 6-bit codes (bit streams, which
// the 4-row kernel's whole-word operands do not read).
static bool only_decode16(const Store &s) {
    return s.bits != 0 && (s.Dk == 96 || s.Dk == 192 || (s.bits != 4 && s.bits != 8));
}

Plan plan_for(const AttendArgs &a) {
    Plan p;
    p.tiles_total = (a.slots + TILE - 1) / TILE;
    const int R = (a.Hq / a.Hkv) * a.L;
    p.rg = R <= 4 ? 1 : (R <= 8 ? 2 : 4);
    const int BH = a.st.BH;
    // Spans are sized so that all workgroups are resident at once (2 per CU): every
    // wavefront streams for the whole kernel and no second scheduling round leaves CUs
    // idle.  A span is a multiple of WAVES tiles so each wavefront gets the same share.
    // (the full-precision kernel, whose tiles are 4x larger, measured faster with one
    // workgroup per CU: 46 us against 52 us at 8192 tokens, B8, 8 kv heads, D 128)
    int want = (a.st.bits != 0 ? 256 * 2 : 256) / BH;
    if (want < 1) want = 1;
    int per = (p.tiles_total + want - 1) / want;
    // KVHIP_DECODE_TILES forces the span size in tiles (timing builds only: measure_knob)
    static const int forced_tiles = measure_knob("KVHIP_DECODE_TILES", 0);
    if (forced_tiles > 0) per = forced_tiles;
    // short sequences (up to 1024 quantized or 512 full-precision rows): one span per pair, so the
    // kernel writes the output rows itself and the merge launch, which costs more than the split
    // gains at this size, is not needed (B1, 4 kv heads, 640 rows, 8-bit: 19.5 -> 16.8 us per step)
    else if (p.tiles_total <= (a.st.bits != 0 ? 4 * WAVES : 2 * WAVES)) per = p.tiles_total;
    per = per < WAVES ? WAVES : per;
    per = (per + WAVES - 1) / WAVES * WAVES;
    while ((p.tiles_total + per - 1) / per > 512) per *= 2;  // the merge kernel holds 512 span weights
    p.tiles_per_wg = per;
    p.nsplit = (p.tiles_total + per - 1) / per;
    // ragged batches (per-batch bounds): the same number of spans for every batch row, each
    // row's visible range divided among them in the kernel (all workgroups stay resident
    // and none is empty; measured faster than equal-sized spans with more of them for the
    // long rows, and than one span size for the whole batch with a row taking as many span slots
    // as its length needs: 37.8 against 42.1 us for B16 U[1024, 16384] at 4 bits, 53.8 against
    // 61.1 us with every row full).  The division needs slots in presented order: a ring
    // presented through a row map keeps equal spans over all of its slots.
    p.nw = WAVES;
    const bool ident = a.runs.n == 1 && a.runs.row0[0] == 0 && a.runs.phys0[0] == 0;
    if (a.mask.mode == KVHIP_MASK_WINDOW && (a.mask.left_pad || a.mask.lengths) && forced_tiles <= 0 && ident) {
        p.tiles_per_wg = 0;
        // KVHIP_RAGGED_SPANS forces the number of spans per batch row (timing builds only: measure_knob)
        static const int forced_spans = measure_knob("KVHIP_RAGGED_SPANS", 0);
        if (forced_spans > 0) p.nsplit = std::min(forced_spans, 512);
    } else if (a.st.bits != 0 && p.nsplit >= 2 && want <= 4 && p.rg == 1 && !only_decode16(a.st) && a.mask.mode != KVHIP_MASK_ARRAY &&
               forced_tiles <= 0) {
        // 128 pairs or more: workgroups of 8 wavefronts, one per CU -- the same wavefronts per CU
        // with half the spans.  With 256 pairs a workgroup takes its pair's whole sequence: the
        // merge stays on chip and the kernel writes the output itself (no partials, no second
        // launch).  Measured at 32k tokens, 4-bit, D 128: B32 207 -> 204 us, B16 112 -> 107 us.
        p.nw = 2 * WAVES;
        int w8 = 256 / BH;
        if (w8 < 1) w8 = 1;
        int per8 = (p.tiles_total + w8 - 1) / w8;
        per8 = (per8 + p.nw - 1) / p.nw * p.nw;
        p.tiles_per_wg = per8;
        p.nsplit = (p.tiles_total + per8 - 1) / per8;
    }
    // a caller with a fixed amount of scratch: fewer, longer spans until the partials fit (one span has none)
    if (a.workspace_cap) {
        const size_t per_span = (size_t)BH * (a.st.bits != 0 && (p.rg >= 2 || only_decode16(a.st)) ? 16 : 4 * p.rg) *
                                (a.st.Dv + 2) * sizeof(float);
        while (p.nsplit > 1 && per_span * p.nsplit > a.workspace_cap) {
            if (p.tiles_per_wg > 0) {
                p.tiles_per_wg *= 2;
                p.nsplit = (p.tiles_total + p.tiles_per_wg - 1) / p.tiles_per_wg;
            } else {
                p.nsplit /= 2;
            }
        }
    }
    return p;
}

// (per calling thread: a thread brackets and reads its own launches)
thread_local int g_profile = 0;        // 0 off, n: bracket every n-th launch of the dominant kernel
thread_local int g_profile_count = 0;  // launches seen since it was enabled
thread_local bool g_profile_open = false;
thread_local std::vector<hipEvent_t> g_events;  // begin/end pairs

}  // namespace

void profile_enable(int every) {
    g_profile = every > 0 ? every : 0;
    g_profile_count = 0;
    g_profile_open = false;
}

void profile_mark(hipStream_t s, bool begin) {
    if (!g_profile) return;
    if (begin) {
        g_profile_open = (g_profile_count++ % g_profile) == 0;
        if (!g_profile_open) return;
    } else if (!g_profile_open) {
        return;
    }
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, s);
    g_events.push_back(e);
}

hipError_t profile_read(int *launches, double *total_ms) {
    *launches = 0;
    *total_ms = 0.0;
    for (size_t i = 0; i + 1 < g_events.size(); i += 2) {
        hipError_t e = hipEventSynchronize(g_events[i + 1]);
        if (e != hipSuccess) return e;
        float ms = 0.f;
        e = hipEventElapsedTime(&ms, g_events[i], g_events[i + 1]);
        if (e != hipSuccess) return e;
        *total_ms += ms;
        *launches += 1;
    }
    for (hipEvent_t ev : g_events) (void)hipEventDestroy(ev);
    g_events.clear();
    return hipSuccess;
}

hipError_t launch_combine(const AttendArgs &a, int nsplit, int rows, hipStream_t s) {
    const int R = (a.Hq / a.Hkv) * a.L;
    dim3 grid(R, a.st.BH);
    if (rows > 16 && nsplit <= 8 && rows == R) {  // the prefill tiles' parts
        dim3 grid4((R + 3) / 4, a.st.BH);
#define CMBR(D)                                                                                      \
    do {                                                                                             \
        if (a.st.dtype == KVHIP_F16) hipLaunchKernelGGL((combine_rows_kernel<D, 0>), grid4, dim3(256), 0, s, a, nsplit, rows); \
        else hipLaunchKernelGGL((combine_rows_kernel<D, 1>), grid4, dim3(256), 0, s, a, nsplit, rows); \
    } while (0)
        if (a.st.Dv == 64) CMBR(64);
        else if (a.st.Dv == 80) CMBR(80);
        else if (a.st.Dv == 96) CMBR(96);
        else if (a.st.Dv == 128) CMBR(128);
        else CMBR(256);
#undef CMBR
        return hipGetLastError();
    }
#define CMB(D)                                                                                       \
    do {                                                                                             \
        if (a.st.dtype == KVHIP_F16) hipLaunchKernelGGL((combine_kernel<D, 0>), grid, dim3(256), 0, s, a, nsplit, rows); \
        else hipLaunchKernelGGL((combine_kernel<D, 1>), grid, dim3(256), 0, s, a, nsplit, rows);       \
    } while (0)
    // (the partials hold output columns: the head size of the values)
    if (a.st.Dv == 64) CMB(64);
    else if (a.st.Dv == 80) CMB(80);
    else if (a.st.Dv == 96) CMB(96);
    else if (a.st.Dv == 128) CMB(128);
    else CMB(256);
#undef CMB
    return hipGetLastError();
}

bool attend_decode_supported(const AttendArgs &a) {
    const Store &s = a.st;
    if (s.dtype != KVHIP_F16 && s.dtype != KVHIP_BF16) return false;
    // keys of 192 with values of 128 (the multi-head latent attention models): quantized caches, on the 16-row kernel
    const bool mla = s.Dk == 192 && s.Dv == 128 && s.bits != 0;
    if (s.Dk != s.Dv && !mla) return false;
    const int R = (a.Hq / a.Hkv) * a.L;
    if (R > 16) return false;
    // full precision: more than 8 rows (4 at D = 256) are faster on the prefill tile than on further
    // passes of the broadcast contraction (8192 keys, 8 kv heads: B16 D 128 16 rows 104 us against
    // 164 us; B8 D 256 8 rows about 105 us against 133 us)
    if (s.bits == 0) return (s.Dk == 64 || s.Dk == 128 || s.Dk == 256) && R <= (s.Dk == 256 ? 4 : 8);
    if (a.runs.n != 1 || a.runs.row0[0] != 0 || a.runs.phys0[0] != 0) return false;
    if (s.bits != 4 && s.bits != 8) return decode16_stream_shape(s);  // every row count on the 16-row kernel
    if (s.Dk == 64) return s.gs == 32 || s.gs == 64;
    if (s.Dk == 96) return s.gs == 32;  // every row count on the 16-row kernel
    if (mla) return s.gs == 32 || s.gs == 64;  // likewise
    if (s.Dk == 128) return s.gs == 32 || s.gs == 64 || s.gs == 128;
    if (s.Dk == 256) return s.gs == 64 || s.gs == 128;
    return false;
}

// The decode kernels -- the 4-row and the 16-row quantized kernel and the full-precision one --, without a mask, write
// a single-token step's new row themselves.
bool attend_decode_fuses_append(const AttendArgs &a) {
    if (!attend_decode_supported(a) || a.L != 1 || a.mask.mode != KVHIP_MASK_NONE) return false;
    static const bool off = measure_knob("KVHIP_NO_FUSED_APPEND", 0) != 0;  // (timing builds only)
    return !off;
}

// 5..16 rows per kv head of a quantized cache go to the 16x16x32 kernel
// (kvhip_attend_decode16.hip), which always carries 16 rows: measured faster than the 4-row
// broadcast contraction from 8 rows up (B16, 8 kv heads, 8192 tokens: 37 us against 43 us at
// 8 rows, 36 us against 87 us at 16).
// The shapes of only_decode16() take it for every row count.
static bool use_decode16(const AttendArgs &a, const Plan &p) {
    return a.st.bits != 0 && (p.rg >= 2 || only_decode16(a.st));
}

size_t attend_decode_workspace(const AttendArgs &a) {
    const Plan p = plan_for(a);
    const int rows = use_decode16(a, p) ? 16 : 4 * p.rg;
    if (p.nsplit == 1) return 0;  // a single span writes the output rows itself: no partials
    return (size_t)a.st.BH * p.nsplit * rows * (a.st.Dv + 2) * sizeof(float);  // (partials hold output columns)
}

hipError_t launch_attend_decode(const AttendArgs &a_in, hipStream_t s) {
    const AttendArgs &a = a_in;
    const Plan p = plan_for(a);
    const Store &st = a.st;
    dim3 grid(p.nsplit, st.BH), block(WAVES * 64);  // the quantized kernel sets its own block size
    const int mm = a.mask.mode == KVHIP_MASK_NONE ? 0 : (a.mask.mode == KVHIP_MASK_ARRAY ? 2 : 1);
#define DEC_K(BITS, D, GS, DT, RG, MM, NW)                                                                \
    hipLaunchKernelGGL((decode_kernel<BITS, D, GS, DT, RG, MM, NW>), grid, dim3(NW * 64), 0, s, a,        \
                       p.tiles_total, p.tiles_per_wg, p.nsplit)
#define DEC(BITS, D, GS, DT, RG)                                                                          \
    do {                                                                                                  \
        profile_mark(s, true);                                                                            \
        if (p.nw == 2 * WAVES) {                                                                          \
            if (mm == 0) DEC_K(BITS, D, GS, DT, RG, 0, 2 * WAVES);                                        \
            else DEC_K(BITS, D, GS, DT, RG, 1, 2 * WAVES);                                                \
        } else if (mm == 0) {                                                                             \
            DEC_K(BITS, D, GS, DT, RG, 0, WAVES);                                                         \
        } else if (mm == 1) {                                                                             \
            DEC_K(BITS, D, GS, DT, RG, 1, WAVES);                                                         \
        } else {                                                                                          \
            DEC_K(BITS, D, GS, DT, RG, 2, WAVES);                                                         \
        }                                                                                                 \
        profile_mark(s, false);                                                                           \
        if (p.nsplit > 1)                                                                                 \
            (void)launch_combine(a, p.nsplit, 4 * RG, s);                                                \
    } while (0)
#define DEC_RG(BITS, D, GS, DT) DEC(BITS, D, GS, DT, 1) /* more rows: the 16-row kernel above */
    if (use_decode16(a_in, p)) {
        profile_mark(s, true);
        hipError_t e = launch_attend_decode16(a_in, p.tiles_total, p.tiles_per_wg, p.nsplit, s);
        profile_mark(s, false);
        if (e != hipSuccess) return e;
        if (p.nsplit > 1) return launch_combine(a_in, p.nsplit, 16, s);
        return hipSuccess;
    }
#define DEC_DT(BITS, D, GS)                                \
    do {                                                   \
        if (st.dtype == KVHIP_F16) DEC_RG(BITS, D, GS, 0); \
        else DEC_RG(BITS, D, GS, 1);                       \
    } while (0)
#define DEC_Q(BITS)                                 \
    do {                                            \
        if (st.Dk == 64 && st.gs == 32) DEC_DT(BITS, 64, 32);   \
        else if (st.Dk == 128 && st.gs == 32) DEC_DT(BITS, 128, 32); \
        else if (st.Dk == 64) DEC_DT(BITS, 64, 64); \
        else if (st.Dk == 256 && st.gs == 64) DEC_DT(BITS, 256, 64);  \
        else if (st.Dk == 256) DEC_DT(BITS, 256, 128);                \
        else if (st.gs == 64) DEC_DT(BITS, 128, 64); \
        else DEC_DT(BITS, 128, 128);                \
    } while (0)
    const bool ident = a.runs.n == 1 && a.runs.row0[0] == 0 && a.runs.phys0[0] == 0;
#define FP(D, DT, RG, M, I)                                                                               \
    do {                                                                                                  \
        profile_mark(s, true);                                                                            \
        hipLaunchKernelGGL((decode_fp_kernel<D, DT, RG, M, I>), grid, block, 0, s, a, p.tiles_total,      \
                           p.tiles_per_wg, p.nsplit);                                                     \
        profile_mark(s, false);                                                                           \
        if (p.nsplit > 1)                                                                                 \
            (void)launch_combine(a, p.nsplit, 4 * RG, s);                                                \
    } while (0)
#define FP_MI(D, DT, RG)                                          \
    do {                                                          \
        if (mm == 0 && ident) FP(D, DT, RG, 0, true);             \
        else if (mm == 0) FP(D, DT, RG, 0, false);                \
        else if (mm == 1 && ident) FP(D, DT, RG, 1, true);        \
        else if (mm == 1) FP(D, DT, RG, 1, false);                \
        else if (ident) FP(D, DT, RG, 2, true);                   \
        else FP(D, DT, RG, 2, false);                             \
    } while (0)
    // (up to 8 query rows per kv head, 4 at D = 256: attend_decode_supported() sends more to the prefill tile)
#define FP_RG(D, DT)                                           \
    do {                                                       \
        if (p.rg == 1) FP_MI(D, DT, 1);                        \
        else if (p.rg == 2 && D < 256) FP_MI(D, DT, (D < 256 ? 2 : 1)); \
        else return hipErrorInvalidValue;                      \
    } while (0)
#define FP_DT(D)                                  \
    do {                                          \
        if (st.dtype == KVHIP_F16) FP_RG(D, 0);   \
        else FP_RG(D, 1);                         \
    } while (0)
    if (st.bits == 4) DEC_Q(4);
    else if (st.bits == 8) DEC_Q(8);
    else if (st.Dk == 64) FP_DT(64);
    else if (st.Dk == 128) FP_DT(128);
    else FP_DT(256);
#undef FP_DT
#undef FP_RG
#undef FP_MI
#undef FP
#undef DEC_Q
#undef DEC_DT
#undef DEC_RG
#undef DEC
#undef DEC_K
    return hipGetLastError();
}

}  // namespace kvhip
