// Chunked-prefill attention for quantized caches on the matrix cores (gfx950,
// v_mfma_f32_16x16x32_f16), head sizes 64 / 96 / 128 / 256 and keys of 192 with values of 128, every code width,
// group size 32 and up.
//
// The loop is the one of the full-precision tile (kvhip_attend_prefill_fp.hip): a workgroup of 4
// wavefronts owns 64 query rows of one (batch, kv-head) pair (QT = 1: 16 per wavefront), or one of 8
// wavefronts 256 rows (QT = 2: 32 per wavefront, head size 128), and walks the keys in tiles of 32, S^T = K . Q^T and out^T += V^T . P^T with K and V tiles double-buffered in LDS,
// software-pipelined so that the scores of tile t + 1 are issued between the exp2 / rounding steps
// of tile t's softmax, one barrier per tile.  What differs is how a tile gets into LDS.  The
// full-precision tile loads it from global memory straight into LDS; here the packed codes are
// loaded into registers one iteration ahead (16 bytes per thread and unit: a K unit is 16 bytes of one
// token's row, a V unit 16 bytes of one column's tile row), turned into float16 values
// scale * code + bias by packed arithmetic (a code OR-ed into the mantissa of a float16 constant is
// that constant plus the code; one packed subtraction and one packed multiply-add per two codes)
// and written to the LDS layout the matrix-core operands are read from -- the vector-ALU work of
// it placed between the out^T matrix-core instructions, whose operands are already in registers.
//   K buffer: [8-element chunk cc][position pos][8 x f16]; position pos holds token
//             8 (pos & 15) / 4 + 4 (pos / 16) + pos % 4 rotated by rot(cc) positions inside its
//             row of 32, so that both the writes (16 lanes: a few tokens x all chunks of a unit) and
//             the operand reads (16 lanes: 16 positions of one chunk) fall on 64 different banks.
//             Inside a chunk the elements come in the order the masked words yield them; the query
//             operands are permuted the same way.
//   V buffer: [8-token chunk tc][column][8 x f16], as in the full-precision tile.
//   (scale, bias) of the V rows: a small LDS table per tile parity, written one iteration before the
//             V tile that needs it is converted.
// Rounding points follow the reference's unfused sequence (KVCache.swift:2351-2447): q * scale
// rounded to T, scores rounded to T, masked scores take finfo(T).min (so a query row that sees no
// key at all averages V over every key); the probabilities are float16 for the matrix cores.
#pragma once

#include <type_traits>

#include "kvhip_mask.hpp"

#ifndef KV_SB
#define KV_SB __builtin_amdgcn_sched_barrier(0)
#endif
namespace kvhip {

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
union Op8 {
    h8 h;
    u4 v;
};

constexpr int BN = 32;  // key slots per tile
constexpr float LOG2E = 1.4426950408889634f;
constexpr float RAISE = 8.f;  // log2 units

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// two codes sitting in the mantissas of a float16 pair (constant + code) -> scale * code + bias
__device__ __forceinline__ uint32_t deq_pair(uint32_t x_bits, kv_h2 magic, kv_h2 sc, kv_h2 bi) {
    kv_h2 x = __builtin_bit_cast(kv_h2, x_bits);
    x = x - magic;
    x = __builtin_elementwise_fma(x, sc, bi);
    return __builtin_bit_cast(uint32_t, x);
}
// position p of a K chunk holds element k_perm(p) of the chunk's 8
template <int BITS> __device__ __forceinline__ constexpr int k_perm(int p) {
    return BITS == 4 ? ((p >> 1) + 4 * (p & 1)) : (BITS == 8 ? ((p & 4) | ((p & 2) >> 1) | ((p & 1) << 1)) : p);
}
// (scale, bias) pair of dtype DT in one dword -> float16 (scale, scale) and (bias, bias)
template <int DT> __device__ __forceinline__ void sb_h2(uint32_t raw, kv_h2 &s2, kv_h2 &b2) {
    if constexpr (DT == 0) {
        s2 = __builtin_bit_cast(kv_h2, __builtin_amdgcn_perm(raw, raw, 0x01000100u));
        b2 = __builtin_bit_cast(kv_h2, __builtin_amdgcn_perm(raw, raw, 0x03020302u));
    } else {
        const _Float16 s = (_Float16)__uint_as_float(raw << 16), b = (_Float16)__uint_as_float(raw & 0xffff0000u);
        s2 = kv_h2{s, s};
        b2 = kv_h2{b, b};
    }
}

// NW wavefronts per workgroup: 4 (two workgroups per CU), or 8 (one per CU; 256 query rows share every
// converted tile, which halves the conversion work per matrix-core instruction)
template <int BITS, int DK, int DV, int DT, int QT, int MM, int NW = 4>
__global__ void __launch_bounds__(64 * NW, NW == 4 ? 2 : 1)
prefill_q_kernel(AttendArgs a, int nsplit) {
    constexpr int NT = 64 * NW;  // threads
    static_assert(BITS == 2 || BITS == 3 || BITS == 4 || BITS == 5 || BITS == 6 || BITS == 8, "affine code widths");
    // 2-, 3-, 5- and 6-bit codes: a row (and a V tile row) is a little-endian bit stream, code j at bit j BITS; a unit
    // is 32 codes (4 BITS bytes), its codes are cut out one by one (bit-field extracts) and paired in natural order
    constexpr bool GEN = BITS != 4 && BITS != 8;
    static_assert((DK == DV && (DK == 64 || DK == 96 || DK == 128 || DK == 256)) || (DK == 192 && DV == 128), "head sizes");
    constexpr int BM = 16 * QT * NW;
    constexpr bool TIGHT = (NW == 8 && QT == 2) || DK >= 256;  // the shapes that have no registers to spare
    constexpr int S = DK / 32;    // contraction steps over the keys' head dim
    constexpr int NDT = DV / 16;  // 16-row tiles of out^T
    constexpr int KSZ = BN * DK, VSZ = BN * DV;  // 16-bit elements of a tile's K and of its V
    // units of UB bytes of packed codes: per tile UK for K (token-major: UPR per token row) and UV for V.
    // 16 bytes, or 8 where that gives every thread of the workgroup a unit (4-bit codes on 8 wavefronts at D <= 128)
    constexpr int UB = GEN ? 4 * BITS : ((32 * (DK + DV) * BITS / 8) / 16 < NT ? 8 : 16);
    constexpr int UWD = UB / 4;                // words per unit
    constexpr int UK = 32 * DK * BITS / 8 / UB, UPR = DK * BITS / 8 / UB, UV = 32 * DV * BITS / 8 / UB;
    constexpr int NU = (UK + UV + NT - 1) / NT;  // units per thread
    constexpr int CPU = UB * 8 / BITS / 8;     // 8-element chunks a unit yields
    constexpr int TOK16 = 16 / UPR > 0 ? 16 / UPR : 1;  // tokens that 16 adjacent lanes of a K write cover
    __shared__ __attribute__((aligned(16))) uint16_t KV0[KSZ + VSZ], KV1[KSZ + VSZ];
    // (scale, bias) of a tile's V rows as float16, two tokens to a word: [tile parity][scale, bias][group][token pair]
    __shared__ __attribute__((aligned(16))) uint32_t tab[2][2][8][BN / 2];
    auto Ks = [&](int par) __attribute__((always_inline)) -> uint16_t * { return par == 0 ? KV0 : KV1; };
    auto Vs = [&](int par) __attribute__((always_inline)) -> uint16_t * { return (par == 0 ? KV0 : KV1) + KSZ; };

    const Store &st = a.st;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, jj = lane >> 4;
    const int G = DV / st.gs;  // groups per V row (1 .. 8)
    // workgroup ids -> (query block, pair, key-range part): all query blocks of a pair on one XCD (one L2)
    const int r = a.Hq / a.Hkv;
    const int R = r * a.L;
    const int nblk = (R + BM - 1) / BM;
    int blk_x, bh, split;
    {
        const int id = blockIdx.x;
        const int BH = st.BH;
        if ((BH & 7) == 0) {
            const int xcd = id & 7;
            int j = id >> 3;
            // (a grid of exactly two workgroups per CU under a causal or window mask: the two workgroups of a CU,
            // 32 apart among the 64 of their XCD, take a long and a short query block)
            if (MM == 1 && gridDim.x == 512 && (j & 32)) j = 95 - j;
            const int per_pair = nblk * nsplit;
            const int h_local = j / per_pair, rem = j - h_local * per_pair;
            bh = h_local * 8 + xcd;
            split = rem / nblk;
            blk_x = rem - split * nblk;
        } else {
            blk_x = id % nblk;
            const int t = id / nblk;
            bh = t % BH;
            split = t / BH;
        }
    }
    // under a causal or window mask the later query blocks see more keys: they get the lower ids, which start first
    if (MM == 1) blk_x = nblk - 1 - blk_x;
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int row0 = blk_x * BM + wave * 16 * QT;  // first query row of this wavefront
    const SymMask sym = sym_mask_init(a.mask, b, a.L, a.T);
    // masked scores take finfo(T).min.  bfloat16: -2^99 stands in for it -- times log2 e it is still finite and the
    // product is exact, so a row of nothing but masked keys gets exactly equal weights, as with the reference's value
    const float fill = DT == 1 ? -0x1p99f : finfo_min_dt(DT);
    // scores enter the softmax as exp2(x - m), x = round_T(s) * log2 e; under an array mask the mask step leaves x
    const float ef = MM == 2 ? 1.f : LOG2E;

    // ---- query operands: B of S^T = K . Q^T; lane (n, jj) holds T(q * scale)[row][32 s + 8 jj ..], chunk order ----
    Op8 qop[QT][S];
    int q_l[QT], q_h[QT];
    bool q_ok[QT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int i = row0 + 16 * qt + n;
        q_ok[qt] = i < R;
        const int rep = q_ok[qt] ? i / a.L : 0;
        q_l[qt] = q_ok[qt] ? i - rep * a.L : 0;
        q_h[qt] = hk * r + rep;
        // rows past R read row (rep 0, l 0), which is in bounds, and are zeroed
        const u4 *qp = reinterpret_cast<const u4 *>(
            reinterpret_cast<const uint16_t *>(a.q) + ((size_t)(b * a.Hq + q_h[qt]) * a.L + q_l[qt]) * DK + 8 * jj);
        u4 raw[S];
#pragma unroll
        for (int s = 0; s < S; ++s) raw[s] = qp[4 * s];
#pragma unroll
        for (int s = 0; s < S; ++s) {
            float qv[8];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t pair = raw[s][w];
                const float v0 = DT == 0 ? (float)__builtin_bit_cast(_Float16, (uint16_t)pair) : __uint_as_float(pair << 16);
                const float v1 = DT == 0 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(pair >> 16)) : __uint_as_float(pair & 0xffff0000u);
                qv[2 * w] = q_ok[qt] ? round_dt<DT>(v0 * a.scale) : 0.f;
                qv[2 * w + 1] = q_ok[qt] ? round_dt<DT>(v1 * a.scale) : 0.f;
            }
#pragma unroll
            for (int w = 0; w < 4; ++w) qop[qt][s].v[w] = pk_h2(qv[k_perm<BITS>(2 * w)], qv[k_perm<BITS>(2 * w + 1)]);
        }
    }

    f4 oacc[QT][NDT];
    float m_run[QT], l_run[QT];
    // the denominators ride on the matrix cores up to D = 128 (lacc = ones . P^T sums the rounded probabilities
    // the numerator uses); D = 256 has no registers to spare
    constexpr bool LM = DV <= 128;
    f4 lacc[LM ? QT : 1];
    Op8 ones;
    ones.v = u4{0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        m_run[qt] = -INFINITY;
        l_run[qt] = 0.f;
        if (LM) lacc[LM ? qt : 0] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) oacc[qt][dt] = f4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- key tiles this workgroup has to visit, and the rows all of its queries keep ---------
    int v_lo = 0, v_hi = (a.slots + BN - 1) / BN;
    int keep_lo = 0, keep_hi = -1;
    {
        const int i_first = blk_x * BM, i_last = min(R, i_first + BM) - 1;
        const bool spans = (i_first / a.L) != (i_last / a.L);
        const int l_min = spans ? 0 : i_first % a.L, l_max = spans ? a.L - 1 : i_last % a.L;
        if (MM != 2) {
            keep_hi = a.T - 1;
            if (MM == 1) {
                if (sym.mode == KVHIP_MASK_CAUSAL) {
                    keep_hi = a.T - a.L + l_min;
                } else {
                    keep_lo = sym.pad_b;
                    keep_hi = min(sym.offset + l_min, sym.len_b - 1);
                    if (sym.window > 0) keep_lo = max(keep_lo, sym.offset + l_max - sym.window + 1);
                }
                keep_hi = min(keep_hi, a.T - 1);
            }
        }
        if (a.mask.mode == KVHIP_MASK_CAUSAL) {
            v_hi = min(v_hi, (a.T - a.L + l_max) / BN + 1);
        } else if (a.mask.mode == KVHIP_MASK_WINDOW) {
            v_hi = min(v_hi, (a.mask.offset + l_max) / BN + 1);
            if (a.mask.window > 0) v_lo = max(0, (a.mask.offset + l_min - a.mask.window + 1) / BN);
        }
        v_hi = min(v_hi, (a.T + BN - 1) / BN);
        if (MM == 1 && sym_mask_some_row_empty(sym)) {  // a fully masked row averages over every key
            v_lo = 0;
            v_hi = (a.T + BN - 1) / BN;
        }
    }
    // optional split of the key range (small grids): each part leaves an unnormalised partial per query row
    if (nsplit > 1) {
        const int span = (v_hi - v_lo + nsplit - 1) / nsplit;
        v_lo = v_lo + split * span;
        v_hi = min(v_hi, v_lo + span);
    }

    // ---- units of packed codes: requests into registers, conversion into LDS ---------------------
    // unit u = tid + NT e: a K unit (u < UK: token u / UPR, part u % UPR of its row) or a V unit
    // (u - UK = h * DV + column: the h-th UB bytes of the column's 32-token half of a tile row)
    uint32_t codes[NU][UWD];
    uint32_t ksb[NU];
    uint32_t vsb_raw[2] = {0u, 0u};  // table entries of a token pair (threads below 16 G)
#pragma unroll
    for (int e = 0; e < NU; ++e) {
#pragma unroll
        for (int w = 0; w < UWD; ++w) codes[e][w] = 0u;
        ksb[e] = 0;
    }
    const size_t cell_k = (size_t)bh * st.k_cell, cell_v = (size_t)bh * st.v_cell;
    const size_t cell_ksb = (size_t)bh * st.ksb_cell, cell_vsb = (size_t)bh * st.vsb_cell;
    PageCursor page_k(st, min(v_lo * BN, max(a.slots - 1, 0))), page_v = page_k;
    auto unit_is_k = [&](int e) __attribute__((always_inline)) -> bool { return tid + NT * e < UK; };
    // Everything about a thread's units that does not change from tile to tile is worked out once (group sizes
    // are powers of two: shifts, no divisions in the loop): byte offsets of the unit's (scale, bias) word and of
    // its V codes in global memory, of its first chunk in the LDS buffer, and of its table row.
    const int gsh = __builtin_ctz((unsigned)st.gs);
    uint32_t u_goff[NU], u_lds[NU], u_tab[NU];
#pragma unroll
    for (int e = 0; e < NU; ++e) {
        const int u = tid + NT * e;
        if (u < UK) {
            const int token = u / UPR, part = u % UPR;
            const int pos = 16 * ((token >> 2) & 1) + 4 * (token >> 3) + (token & 3);
            u_goff[e] = (uint32_t)token * st.ksb_row + (uint32_t)(((part * (UB * 8 / BITS)) >> gsh) * 4);
            u_lds[e] = (uint32_t)(((part * CPU) * BN + ((pos + TOK16 * part) & (BN - 1))) * 16);
            u_tab[e] = 0;
        } else {
            const int uv = u - UK, d = uv % DV, h = uv / DV;
            u_goff[e] = (uint32_t)(d * (TILE * BITS / 8) + h * UB);
            u_lds[e] = (uint32_t)(((h * CPU) * DV + d) * 16);
            u_tab[e] = (uint32_t)(((d >> gsh) * (BN / 2) + 4 * h * CPU) * 4);
        }
    }
    const bool tab_thread = tid < (BN / 2) * G;  // (G = 3 at head size 96: a division, once)
    const int tab_tp = tid / G, tab_g = tid - tab_tp * G;
    const uint32_t tab_goff0 = (uint32_t)(2 * tab_tp * G + tab_g) * 4u;  // (the pair's second token: one row of G words further)
    auto unit_is_v = [&](int e) __attribute__((always_inline)) -> bool { return tid + NT * e >= UK && tid + NT * e < UK + UV; };
    auto load_unit = [&](uint32_t (&dst)[UWD], gptr p) __attribute__((always_inline)) {
        if constexpr (GEN) {  // 4-byte aligned: words one by one
#pragma unroll
            for (int w = 0; w < UWD; ++w) dst[w] = ld_global<uint32_t>(p, w);
        } else if constexpr (UWD == 4) {
            const u4 v = ld_global<u4>(p);
            dst[0] = v.x;
            dst[1] = v.y;
            dst[2] = v.z;
            dst[3] = v.w;
        } else {
            const kv_u2 v = ld_global<kv_u2>(p);
            dst[0] = v.x;
            dst[1] = v.y;
        }
    };
    // tile_k: codes and (scale, bias) of the K units and the table entry of the V rows; tile_v: codes of the V units
    auto request = [&](int tile_k, bool do_k, int tile_v, bool do_v) __attribute__((always_inline)) {
        if (do_k) {
            const int slot0 = tile_k * BN, in_page = slot0 & (PAGE - 1);
            const PageEntry &pe = page_k.at(st, slot0);
            gptr kb = as_global(pe.k + cell_k + (size_t)in_page * st.k_row);
            gptr sbb = as_global(pe.ksb + cell_ksb + (size_t)in_page * st.ksb_row);
#pragma unroll
            for (int e = 0; e < NU; ++e)
                if (unit_is_k(e)) {
                    // (TIGHT: the 32-bit lane offsets are handed over as they are -- held across the loop the compiler
                    // keeps each as a zero-extended 64-bit pair, twice the registers, and spills them)
                    uint32_t ko = (uint32_t)((tid + NT * e) * UB), go = u_goff[e];
                    if constexpr (TIGHT) asm volatile("" : "+v"(ko), "+v"(go));
                    load_unit(codes[e], kb + ko);  // the tile's K rows are one contiguous block
                    ksb[e] = ld_global<uint32_t>(sbb + go);
                }
            if (tab_thread) {  // thread (token pair, group): the two tokens' (scale, bias) words
                gptr vsbb = as_global(pe.vsb + cell_vsb + (size_t)in_page * st.vsb_row);
                uint32_t t0 = tab_goff0;
                if constexpr (TIGHT) asm volatile("" : "+v"(t0));
                vsb_raw[0] = ld_global<uint32_t>(vsbb + t0);
                vsb_raw[1] = ld_global<uint32_t>(vsbb + t0 + 4u * (uint32_t)G);
            }
        }
        if (do_v) {
            const int slot0 = tile_v * BN;
            const PageEntry &pe = page_v.at(st, slot0);
            gptr vb = as_global(pe.v + cell_v + (size_t)((slot0 & (PAGE - 1)) >> 6) * DV * (TILE * BITS / 8) +
                                ((slot0 & 32) ? BN * BITS / 8 : 0));
#pragma unroll
            for (int e = 0; e < NU; ++e)
                if (unit_is_v(e)) {
                    uint32_t go = u_goff[e];
                    if constexpr (TIGHT) asm volatile("" : "+v"(go));
                    load_unit(codes[e], vb + go);
                }
        }
    };
    // the table of the V rows' (scale, bias) pairs of the tile whose entry `request` fetched
    auto write_table = [&](int par) __attribute__((always_inline)) {
        if (tab_thread) {
            const int tp = tab_tp, g = tab_g;
            uint32_t w0 = vsb_raw[0], w1 = vsb_raw[1];
            if constexpr (DT == 1) {  // bfloat16 pairs -> float16 pairs
                w0 = pk_h2(__uint_as_float(w0 << 16), __uint_as_float(w0 & 0xffff0000u));
                w1 = pk_h2(__uint_as_float(w1 << 16), __uint_as_float(w1 & 0xffff0000u));
            }
            tab[par][0][g][tp] = __builtin_amdgcn_perm(w1, w0, 0x05040100u);  // (scale of the even token, of the odd one)
            tab[par][1][g][tp] = __builtin_amdgcn_perm(w1, w0, 0x07060302u);  // (bias, bias)
        }
    };
    const kv_h2 m1024 = kv_h2{(_Float16)1024.f, (_Float16)1024.f}, m64 = kv_h2{(_Float16)64.f, (_Float16)64.f};
    // The float16 constants the codes are OR-ed into, held in vector registers the compiler cannot rematerialise:
    // (w & mask) | constant is then one v_and_or_b32 (mask in a scalar register, constant in a vector register; with
    // both as literals the instruction, which may read one scalar operand, is not formed), and an 8-bit pair is one
    // v_perm_b32 that takes bytes 0 and 2 (or 1 and 3) of the word beside the constant's high bytes.
    uint32_t mag = 0x64006400u, mag_hi = 0x54005400u;
    asm volatile("" : "+v"(mag), "+v"(mag_hi));
    auto nib_lo = [&](uint32_t w) __attribute__((always_inline)) -> uint32_t { return (w & 0x000f000fu) | mag; };
    auto nib_hi = [&](uint32_t w) __attribute__((always_inline)) -> uint32_t { return (w & 0x00f000f0u) | mag_hi; };
    auto bytes_even = [&](uint32_t w) __attribute__((always_inline)) -> uint32_t { return __builtin_amdgcn_perm(mag, w, 0x05020500u); };
    auto bytes_odd = [&](uint32_t w) __attribute__((always_inline)) -> uint32_t { return __builtin_amdgcn_perm(mag, w, 0x05030501u); };
    // chunk c (0 .. CPU-1) of K unit e -> LDS
    auto convert_k = [&](int e, int c, int par) __attribute__((always_inline)) {
        kv_h2 s2, b2;
        sb_h2<DT>(ksb[e], s2, b2);
        u4 o;
        if constexpr (GEN) {
            const u4 x = stream_chunk<BITS, UWD>(codes[e], c, mag);
            o.x = deq_pair(x.x, m1024, s2, b2);
            o.y = deq_pair(x.y, m1024, s2, b2);
            o.z = deq_pair(x.z, m1024, s2, b2);
            o.w = deq_pair(x.w, m1024, s2, b2);
        } else if constexpr (BITS == 4) {  // elements (0,4) (1,5) (2,6) (3,7) of the word's 8
            const uint32_t w = codes[e][c], w8 = w >> 8;
            o.x = deq_pair(nib_lo(w), m1024, s2, b2);
            o.y = deq_pair(nib_hi(w), m64, s2, b2);
            o.z = deq_pair(nib_lo(w8), m1024, s2, b2);
            o.w = deq_pair(nib_hi(w8), m64, s2, b2);
        } else {  // elements (0,2) (1,3) of each word's 4
            const uint32_t w0 = codes[e][2 * c], w1 = codes[e][2 * c + 1];
            o.x = deq_pair(bytes_even(w0), m1024, s2, b2);
            o.y = deq_pair(bytes_odd(w0), m1024, s2, b2);
            o.z = deq_pair(bytes_even(w1), m1024, s2, b2);
            o.w = deq_pair(bytes_odd(w1), m1024, s2, b2);
        }
        *reinterpret_cast<u4 *>(reinterpret_cast<char *>(Ks(par)) + u_lds[e] + c * (BN * 16)) = o;
    };
    // chunk c of V unit e -> LDS (tpar: the parity of the table of this tile)
    auto convert_v = [&](int e, int c, int par) __attribute__((always_inline)) {
        // chunk c of the unit: tokens 8 tc .. 8 tc + 7 of the tile, tc = h CPU + c
        const char *trow = reinterpret_cast<const char *>(&tab[par][0][0][0]) + u_tab[e] + c * 16;
        const u4 sv = *reinterpret_cast<const u4 *>(trow);
        const u4 bv = *reinterpret_cast<const u4 *>(trow + sizeof(tab[0][0]));
        // (the words go through scalars first: a bit cast applied to a vector element expression reads element 0)
        const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
        const kv_h2 s0 = __builtin_bit_cast(kv_h2, sw[0]), s1 = __builtin_bit_cast(kv_h2, sw[1]);
        const kv_h2 s2 = __builtin_bit_cast(kv_h2, sw[2]), s3 = __builtin_bit_cast(kv_h2, sw[3]);
        const kv_h2 b0 = __builtin_bit_cast(kv_h2, bw[0]), b1 = __builtin_bit_cast(kv_h2, bw[1]);
        const kv_h2 b2 = __builtin_bit_cast(kv_h2, bw[2]), b3 = __builtin_bit_cast(kv_h2, bw[3]);
        u4 o;
        if constexpr (GEN) {  // a plain bit stream over the tile's tokens
            const u4 x = stream_chunk<BITS, UWD>(codes[e], c, mag);
            o.x = deq_pair(x.x, m1024, s0, b0);
            o.y = deq_pair(x.y, m1024, s1, b1);
            o.z = deq_pair(x.z, m1024, s2, b2);
            o.w = deq_pair(x.w, m1024, s3, b3);
        } else if constexpr (BITS == 4) {  // the word's tokens two at a time, in token order (the V tile's nibble order)
            const uint32_t w = codes[e][c], w8 = w >> 8;
            o.x = deq_pair(nib_lo(w), m1024, s0, b0);
            o.y = deq_pair(nib_hi(w), m64, s1, b1);
            o.z = deq_pair(nib_lo(w8), m1024, s2, b2);
            o.w = deq_pair(nib_hi(w8), m64, s3, b3);
        } else {
            const uint32_t w0 = codes[e][2 * c], w1 = codes[e][2 * c + 1];
            o.x = deq_pair(bytes_even(w0), m1024, s0, b0);
            o.y = deq_pair(bytes_odd(w0), m1024, s1, b1);
            o.z = deq_pair(bytes_even(w1), m1024, s2, b2);
            o.w = deq_pair(bytes_odd(w1), m1024, s3, b3);
        }
        *reinterpret_cast<u4 *>(reinterpret_cast<char *>(Vs(par)) + u_lds[e] + c * (DV * 16)) = o;
    };
    // piece p (0 .. NU CPU - 1) of this thread's conversions: K units go to Ks(kpar), V units to Vs(vpar)
    constexpr int NPIECE = NU * CPU;
    auto convert_piece = [&](int p, bool do_k, int kpar, bool do_v, int vpar) __attribute__((always_inline)) {
        const int e = p / CPU, c = p % CPU;
        if (do_k && unit_is_k(e)) convert_k(e, c, kpar);
        if (do_v && unit_is_v(e)) convert_v(e, c, vpar);
    };

    // ---- S^T = K . Q^T operands: K slot (chunk 4 s + jj, position 16 mt + n) ------------------------
    // (chunk cc = 4 s + jj is rotated by TOK16 (cc / CPU) positions; CPU divides 4, so that is a per-lane part,
    // TOK16 (jj / CPU), plus a constant of the step.  The eight addresses of an iteration are then three
    // instructions each from two lane constants.  The 256-row shape, which has no registers to keep eight
    // addresses in -- held across the loop they were spilled to scratch memory and reloaded in front of every
    // operand read, on the path to the matrix-core instruction that waits for it -- forms them anew every time.)
    static_assert(4 % CPU == 0, "a contraction step's four chunks are whole units");
    const int k_pos0 = n + TOK16 * (jj / CPU);        // position of this lane's row before the step's rotation
    const int k_byte0 = jj * (BN * 16);               // byte offset of chunk jj
    auto read_k = [&](int par, int s, Op8 (&ka)[2]) __attribute__((always_inline)) {
        int pos0 = k_pos0;
        if constexpr (TIGHT) asm volatile("" : "+v"(pos0));  // (not hoisted out of the loop)
        const char *base = reinterpret_cast<const char *>(Ks(par)) + k_byte0 + s * (4 * BN * 16);
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            const int pos = (pos0 + 16 * mt + TOK16 * (4 / CPU) * s) & (BN - 1);
            ka[mt].v = *reinterpret_cast<const u4 *>(base + pos * 16);
        }
    };

    // ---- mask of the tile at slot0 whose raw scores are in `sc` ------------------------------------
    // lane (n, jj) holds, per query block, the scores of tokens slot0 + 8 jj + 4 mt + i.  Rows past the end
    // become -inf (no weight); rows the mask excludes take `fill`; under an array mask the scores are
    // rounded and moved to the log2 domain here
    [[maybe_unused]] int q_lo[QT];
    [[maybe_unused]] uint32_t q_span[QT];
    if constexpr (MM == 1) {
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            int lo, hi;
            if (sym.mode == KVHIP_MASK_CAUSAL) {
                lo = 0;
                hi = a.T - a.L + q_l[qt];
            } else {
                const int li = sym.offset + q_l[qt];
                lo = sym.pad_b;
                hi = min(li, sym.len_b - 1);
                if (sym.window > 0) lo = max(lo, li - sym.window + 1);
            }
            lo = max(lo, 0);
            hi = min(hi, a.T - 1);
            const bool any = hi >= lo;
            q_lo[qt] = any ? lo : 0x40000000;  // (no row reaches it: row - q_lo wraps to a huge unsigned value)
            q_span[qt] = any ? (uint32_t)(hi - lo) : 0u;
        }
    }
    auto apply_mask = [&](int slot0, f4 (&sc)[QT][2]) __attribute__((always_inline)) {
        const int base = slot0 + 8 * jj;
        if constexpr (MM != 2) {
#pragma unroll
            for (int qt = 0; qt < QT; ++qt)
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = base + 4 * mt + i;
                        float v = sc[qt][mt][i];
                        if constexpr (MM == 1) v = ((uint32_t)(row - q_lo[qt]) <= q_span[qt]) ? v : fill;
                        sc[qt][mt][i] = row < a.T ? v : -INFINITY;
                    }
            return;
        } else {
            const bool vec_ok = a.mask.dtype == KVHIP_BOOL;  // a lane's eight rows are consecutive: two words of four keys
#pragma unroll
            for (int qt = 0; qt < QT; ++qt) {
                uint32_t mword[2] = {0u, 0u};
                if (vec_ok && q_ok[qt]) {
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
                        if (base + 4 * mt + 3 < a.T) {
                            uint32_t w[1];
                            mask_bool_words<1>(a.mask, b, q_h[qt], q_l[qt], base + 4 * mt, w);
                            mword[mt] = w[0];
                        }
                }
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = base + 4 * mt + i;
                        float x_ = round_dt<DT>(sc[qt][mt][i]);
                        bool keep = true;
                        if (row < a.T && q_ok[qt]) {
                            if (vec_ok && base + 4 * mt + 3 < a.T) {
                                keep = ((mword[mt] >> (8 * i)) & 0xffu) != 0u;
                            } else {
                                float add;
                                keep = mask_keep(a.mask, b, q_h[qt], q_l[qt], row, a.L, a.T, add);
                                if (a.mask.dtype != KVHIP_BOOL) x_ = round_dt<DT>(x_ + add);
                            }
                        }
                        x_ = keep ? x_ : fill;
                        sc[qt][mt][i] = row < a.T ? x_ * LOG2E : -INFINITY;
                    }
            }
        }
    };

    // ---- tile maximum and the reference maximum (log2 domain; see the full-precision tile) ------------
    auto raise = [&](int qt, float tmax) __attribute__((always_inline)) {
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float mn = fmaxf(m_run[qt], tmax);
        const float alpha = (mn == -INFINITY) ? 1.f : exp2_fast(m_run[qt] - mn);
        m_run[qt] = mn;
        if constexpr (LM) {
#pragma unroll
            for (int i = 0; i < 4; ++i) lacc[LM ? qt : 0][i] *= alpha;
        } else {
            l_run[qt] *= alpha;
        }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) oacc[qt][dt][i] *= alpha;
    };
    auto tile_max = [&](const f4 (&sc)[QT][2], int qt) __attribute__((always_inline)) -> float {
        return ef * fmaxf(fmaxf(fmaxf(sc[qt][0][0], sc[qt][0][1]), fmaxf(sc[qt][0][2], sc[qt][0][3])),
                          fmaxf(fmaxf(sc[qt][1][0], sc[qt][1][1]), fmaxf(sc[qt][1][2], sc[qt][1][3])));
    };
    // The same maximum in four instructions, for the end of an iteration.  `fmaxf` on values the compiler has not
    // seen an arithmetic instruction produce (matrix-core results, selects) first quiets each operand with a
    // maximum of its own: eleven instructions for eight values, on the path every wavefront runs before the
    // barrier.  Written as assembly, which the compiler's hazard handling does not look into: the caller keeps it
    // behind a scheduling barrier that follows the out^T matrix-core instructions, so the score registers, written
    // by matrix-core instructions a whole block earlier (or by the mask's selects), are long complete.
    auto tile_max_raw = [&](const f4 (&sc)[QT][2], int qt) __attribute__((always_inline)) -> float {
        float m;  // (one statement per instruction: the result may then share a register with a finished operand)
        asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(m) : "v"(sc[qt][0][0]), "v"(sc[qt][0][1]), "v"(sc[qt][0][2]));
        asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(m) : "v"(m), "v"(sc[qt][0][3]), "v"(sc[qt][1][0]));
        asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(m) : "v"(m), "v"(sc[qt][1][1]), "v"(sc[qt][1][2]));
        asm volatile("v_max_f32 %0, %1, %2" : "=v"(m) : "v"(m), "v"(sc[qt][1][3]));
        return ef * m;
    };
    auto needs_raise = [&](const f4 (&sc)[QT][2]) __attribute__((always_inline)) -> bool {
        bool need = false;
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) need = need || tile_max_raw(sc, qt) > m_run[qt] + RAISE;
        return __any(need);
    };
    auto do_raise = [&](const f4 (&sc)[QT][2]) __attribute__((always_inline)) {
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            const float tmax = tile_max(sc, qt);
            if (__any(tmax > m_run[qt] + RAISE)) raise(qt, tmax);
        }
    };

    // ---- one iteration: tile position `tile` (parity PAR) has its scores in `sc`; `sn` receives tile + 1's.
    // K(tile + 2) and V(tile + 1), whose codes the previous iteration requested, are converted into the buffers
    // the previous iteration read last; then K(tile + 3) and V(tile + 2) are requested.
    auto body = [&](auto HAS_NEXT_, auto PAR_, auto MASKED_, int tile, f4 (&sc)[QT][2], f4 (&sn)[QT][2], bool &need) __attribute__((always_inline)) {
        constexpr bool HAS_NEXT = decltype(HAS_NEXT_)::value;
        constexpr int PAR = decltype(PAR_)::value;
        constexpr bool MASKED = decltype(MASKED_)::value;
        const bool k2 = tile + 2 < v_hi;

        float negmu[QT], pr[QT][2][4];
        Op8 pb[QT];
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) negmu[qt] = (m_run[qt] == -INFINITY) ? 0.f : -m_run[qt];
        auto round_pair = [&](int idx) __attribute__((always_inline)) {  // idx: the odd member of the pair
            const int qt = idx >> 3, mt = (idx >> 2) & 1, i = idx & 3;
            const float p0 = pr[qt][mt][i - 1], p1 = pr[qt][mt][i];
            if constexpr (!LM) l_run[qt] += p0 + p1;
            pb[qt].v[2 * mt + (i >> 1)] = pk_h2(p0, p1);
        };
        constexpr int NP = 8 * QT;  // probabilities per lane and tile
        auto softmax_slice = [&](int idx) __attribute__((always_inline)) {
            const int qt = idx >> 3, mt = (idx >> 2) & 1, i = idx & 3;
            // the reference rounds the scores to T before the softmax (under an array mask the mask step has done it)
            const float x = MM == 2 ? sc[qt][mt][i] + negmu[qt] : __builtin_fmaf(round_dt<DT>(sc[qt][mt][i]), LOG2E, negmu[qt]);
            pr[qt][mt][i] = exp2_fast(x);  // exp2(-inf) = 0 for keys past the end
            if ((idx & 1) && idx >= 3) round_pair(idx - 2);
            if (idx == NP - 1) round_pair(idx);
        };
        constexpr int VG = 2, NVB = 2;
        constexpr int NG = (NDT + VG - 1) / VG;
        Op8 va[NVB][VG];
        auto read_v = [&](int g, Op8 (&dst)[VG]) __attribute__((always_inline)) {
#pragma unroll
            for (int x = 0; x < VG; ++x)
                if (VG * g + x < NDT)  // tokens 8 jj .. 8 jj + 7 of column 16 (VG g + x) + n: one chunk
                    dst[x].v = *reinterpret_cast<const u4 *>(&Vs(PAR)[(jj * DV + 16 * (VG * g + x) + n) * 8]);
        };
        if (k2) write_table(PAR);  // of tile + 2: this buffer's last reader was the previous iteration
        if constexpr (HAS_NEXT) {
            constexpr int NM = 2 * S * QT;  // matrix-core instructions of the next tile's scores
            constexpr int AHEAD = QT == 1 ? 2 : 1;
            constexpr int KA = S < AHEAD + 1 ? S : AHEAD + 1;
            Op8 ka[KA][2];
#pragma unroll
            for (int s = 0; s < (S < AHEAD ? S : AHEAD); ++s) read_k(PAR ^ 1, s, ka[s % KA]);
            KV_SB;
#pragma unroll
            for (int k = 0; k < NM; ++k) {
                const int s = k / (2 * QT), mt = (k / QT) & 1, qt = k % QT;
                if (k % (2 * QT) == 0 && s + AHEAD < S) read_k(PAR ^ 1, s + AHEAD, ka[(s + AHEAD) % KA]);
                if (k == (NM > 2 * QT ? NM - 2 * QT : 0)) {
#pragma unroll
                    for (int g = 0; g < NVB - 1 && g < NG; ++g) read_v(g, va[g]);
                }
                if (s == 0) sn[qt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[s % KA][mt].h, qop[qt][s].h, f4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                else sn[qt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[s % KA][mt].h, qop[qt][s].h, sn[qt][mt], 0, 0, 0);
#pragma unroll
                for (int idx = k * NP / NM; idx < (k + 1) * NP / NM; ++idx) softmax_slice(idx);
                KV_SB;
            }
        } else {
#pragma unroll
            for (int g = 0; g < NVB - 1 && g < NG; ++g) read_v(g, va[g]);
#pragma unroll
            for (int idx = 0; idx < NP; ++idx) softmax_slice(idx);
        }

        // ---- out^T += V^T . P^T, with this thread's conversions spread between the groups ----
        if constexpr (LM) {
#pragma unroll
            for (int qt = 0; qt < QT; ++qt)
                lacc[LM ? qt : 0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones.h, pb[qt].h, lacc[LM ? qt : 0], 0, 0, 0);
        }
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            if (g + NVB - 1 < NG) read_v(g + NVB - 1, va[(g + NVB - 1) % NVB]);
#pragma unroll
            for (int x = 0; x < VG; ++x)
                if (VG * g + x < NDT) {
#pragma unroll
                    for (int qt = 0; qt < QT; ++qt)
                        oacc[qt][VG * g + x] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[g % NVB][x].h, pb[qt].h, oacc[qt][VG * g + x], 0, 0, 0);
                }
            if constexpr (HAS_NEXT) {
#pragma unroll
                for (int p = g * NPIECE / NG; p < (g + 1) * NPIECE / NG; ++p) convert_piece(p, k2, PAR, true, PAR ^ 1);
            }
        }
        if constexpr (HAS_NEXT) request(tile + 3, tile + 3 < v_hi, tile + 2, k2);

        need = false;
        if constexpr (HAS_NEXT) {
            if constexpr (MASKED) apply_mask((tile + 1) * BN, sn);
            KV_SB;  // (tile_max_raw: not before the matrix-core instructions above)
            need = needs_raise(sn);
        }
        // the conversions' LDS writes have to land before any wavefront reads the buffers
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };

    if (v_lo < v_hi) {
        // K(v_lo), V(v_lo) and K(v_lo + 1) are converted before the loop starts
        request(v_lo, true, v_lo, true);
        write_table(0);
        __syncthreads();
#pragma unroll
        for (int p = 0; p < NPIECE; ++p) convert_piece(p, true, 0, true, 0);
        const bool k1 = v_lo + 1 < v_hi;
        request(v_lo + 1, k1, 0, false);
        if (k1) {
            write_table(1);
#pragma unroll
            for (int p = 0; p < NPIECE; ++p) convert_piece(p, true, 1, false, 0);
        }
        request(v_lo + 2, v_lo + 2 < v_hi, v_lo + 1, k1);
        __syncthreads();
        f4 sa[QT][2], sb[QT][2];
        {  // scores of the first tile
#pragma unroll
            for (int s = 0; s < S; ++s) {
                Op8 ka[2];
                read_k(0, s, ka);
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int qt = 0; qt < QT; ++qt)
                        sa[qt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[mt].h, qop[qt][s].h, s == 0 ? f4{0.f, 0.f, 0.f, 0.f} : sa[qt][mt], 0, 0, 0);
            }
            if (MM == 2 || !(v_lo * BN >= keep_lo && v_lo * BN + (BN - 1) <= keep_hi)) apply_mask(v_lo * BN, sa);
            do_raise(sa);
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // K buffer 0 is free again
        using T_ = std::true_type;
        using F_ = std::false_type;
        using P0 = std::integral_constant<int, 0>;
        using P1 = std::integral_constant<int, 1>;
        int tile = v_lo;
        auto iterate = [&](auto PAR_, f4 (&sc)[QT][2], f4 (&sn)[QT][2], bool &need) __attribute__((always_inline)) -> bool {
            const bool has_next = tile + 1 < v_hi;
            bool masked = true;
            if constexpr (MM != 2) masked = !((tile + 1) * BN >= keep_lo && (tile + 1) * BN + (BN - 1) <= keep_hi);
            if (has_next) {
                if (__builtin_amdgcn_readfirstlane(masked)) body(T_{}, PAR_, T_{}, tile, sc, sn, need);
                else if constexpr (MM != 2) body(T_{}, PAR_, F_{}, tile, sc, sn, need);
                ++tile;
                return true;
            }
            body(F_{}, PAR_, F_{}, tile, sc, sn, need);
            return false;
        };
        for (;;) {
            // the fast loop: two iterations (one per buffer parity) per round, left when a tile's scores call for a
            // higher reference maximum (the accumulators are rescaled outside it: see the full-precision tile)
            bool more = true, need = false, odd = false;
            for (;;) {
                more = iterate(P0{}, sa, sb, need);
                odd = true;
                if (!more || need) break;
                more = iterate(P1{}, sb, sa, need);
                odd = false;
                if (!more || need) break;
            }
            if (!more) break;
            if (odd) {
                do_raise(sb);
                more = iterate(P1{}, sb, sa, need);
                if (!more) break;
                if (need) do_raise(sa);
            } else {
                do_raise(sa);
            }
        }
    }

    // ---- normalise and store: lane (n, jj) holds out[q = n][d = 16 dt + 4 jj + i] ------------
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        float l = l_run[qt];
        if constexpr (LM) {
            l = lacc[LM ? qt : 0][0];
        } else {
            l += __shfl_xor(l, 16);
            l += __shfl_xor(l, 32);
        }
        if (!q_ok[qt]) continue;
        if (nsplit > 1) {
            const int i = row0 + 16 * qt + n;
            float *part = a.workspace + (((size_t)bh * nsplit + split) * R + i) * (DV + 2);
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f4 *>(part + 16 * dt + 4 * jj) = oacc[qt][dt];
            if (jj == 0) {
                part[DV] = m_run[qt] * 0.6931471805599453f;  // back from the log2 domain
                part[DV + 1] = l;
            }
            continue;
        }
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        const size_t ooff = ((size_t)(b * a.Hq + q_h[qt]) * a.L + q_l[qt]) * DV;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            const float o0 = oacc[qt][dt][0] * inv, o1 = oacc[qt][dt][1] * inv;
            const float o2 = oacc[qt][dt][2] * inv, o3 = oacc[qt][dt][3] * inv;
            uint2 w;
            if (DT == 0) {
                w.x = pk_h2(o0, o1);
                w.y = pk_h2(o2, o3);
            } else {
                w.x = pk_bf2(o0, o1);
                w.y = pk_bf2(o2, o3);
            }
            *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(a.out) + ooff + 16 * dt + 4 * jj) = w;
        }
    }
}

// Launch for one code width: `rows` query rows per workgroup -- 64 on 4 wavefronts; keys of 192 with values of 128 also
// 128 on 8 wavefronts (one workgroup per CU, twice as many rows share each converted tile: 454 against 366 TFLOP/s at
// B1, 16 heads, 2048 x 8192, 4 bits; the other head sizes measured no faster or slower that way); WIDE (4- and 8-bit
// codes) at head size 128 also 256 rows on 8 wavefronts.
template <int BITS, bool WIDE>
hipError_t launch_prefill_q_bits(const AttendArgs &a, int nsplit, int rows, hipStream_t s) {
    const Store &st = a.st;
    const int R = (a.Hq / a.Hkv) * a.L;
    if (rows != 64 && !(rows == 128 && st.Dk == 192) && !(WIDE && rows == 256 && st.Dk == 128)) return hipErrorInvalidValue;
    dim3 grid((unsigned)((R + rows - 1) / rows) * st.BH * nsplit), block(rows == 64 ? 256 : 512);
    const int mm = a.mask.mode == KVHIP_MASK_NONE ? 0 : (a.mask.mode == KVHIP_MASK_ARRAY ? 2 : 1);
#define PQ_M(DK, DV, DT, QT, NW)                                                                                 \
    do {                                                                                                         \
        if (mm == 0) hipLaunchKernelGGL((prefill_q_kernel<BITS, DK, DV, DT, QT, 0, NW>), grid, block, 0, s, a, nsplit);      \
        else if (mm == 1) hipLaunchKernelGGL((prefill_q_kernel<BITS, DK, DV, DT, QT, 1, NW>), grid, block, 0, s, a, nsplit); \
        else hipLaunchKernelGGL((prefill_q_kernel<BITS, DK, DV, DT, QT, 2, NW>), grid, block, 0, s, a, nsplit);              \
    } while (0)
#define PQ_DT(DK, DV, QT, NW)                              \
    do {                                                   \
        if (st.dtype == KVHIP_F16) PQ_M(DK, DV, 0, QT, NW); \
        else PQ_M(DK, DV, 1, QT, NW);                      \
    } while (0)
    if (st.Dk == 64) {
        PQ_DT(64, 64, 1, 4);
    } else if (st.Dk == 96) {
        PQ_DT(96, 96, 1, 4);
    } else if (st.Dk == 128) {
        if constexpr (WIDE) {
            if (rows == 256) {
                PQ_DT(128, 128, 2, 8);
                return hipGetLastError();
            }
        }
        PQ_DT(128, 128, 1, 4);
    } else if (st.Dk == 192) {
        if (rows == 128) PQ_DT(192, 128, 1, 8);
        else PQ_DT(192, 128, 1, 4);
    } else {
        PQ_DT(256, 256, 1, 4);
    }
#undef PQ_DT
#undef PQ_M
    return hipGetLastError();
}

}  // namespace
}  // namespace kvhip
