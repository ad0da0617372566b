// Chunked-prefill attention tile on the matrix cores (gfx950, v_mfma_f32_16x16x32_f16) for
// quantized caches of head size 96 and of keys 192 with values 128 (head sizes 64 / 128 / 256 take the
// pipelined tile of kvhip_attend_prefill_q.hip, full-precision caches the kernel of
// kvhip_attend_prefill_fp.hip), and the launcher of all three.
//
// Many query rows per kv head (r = Hq/Hkv heads times L new tokens).  One workgroup
// (4 wavefronts) owns 128 query rows of one (batch, kv-head) pair -- 32 per wavefront
// -- and walks the cached keys in tiles of 32 physical slots.  A tile is staged once
// per workgroup in LDS as fp16 (the packed codes are dequantised here),
// K as [token][d] and V as [d][token], which is how the page layout already stores
// them; the dense contractions then run as
//   S^T   = K . Q^T      A = K rows from LDS, B = query rows held in registers
//   out^T += V^T . P^T   A = V^T rows from LDS, B = the probabilities exactly where the
//                        S^T accumulators left them (lane (q, j) holds tokens 4j..4j+3 of
//                        both 16-token halves), so P never moves between lanes
// with the online softmax in fp32 between them.  Masks are evaluated from indices
// (causal, window, lengths, left padding) or read from the caller's array; for the
// symbolic ones whole key tiles outside the visible range are skipped.
#include <cstdlib>

#include "kvhip_mask.hpp"

namespace kvhip {

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
union Op8 {
    h8 h;
    uint32_t u[4];
    uint2 d2[2];
    uint4 v;
};

constexpr int BN = 32;    // key slots per tile


constexpr float LOG2E = 1.4426950408889634f;
constexpr float RAISE = 5.545177444479562f;  // 8 ln 2

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ uint16_t h_bits(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
__device__ __forceinline__ uint32_t h2_bits(float lo, float hi) { return pk_h2(lo, hi); }

// Codes become float16 values without an integer-to-float conversion: a code OR-ed into the mantissa of a
// float16 constant (1024 for bits 0..9 of the mantissa, 64 for a nibble at bits 4..7) is that constant plus the
// code, exactly; subtracting the constant leaves the code, and one packed multiply-add applies scale and bias
// to two codes at a time (a single rounding to float16, which is what the tile holds in LDS anyway).
__device__ __forceinline__ uint32_t deq_pair(uint32_t masked_or_magic, kv_h2 magic, kv_h2 sc, kv_h2 bi) {
    kv_h2 x = __builtin_bit_cast(kv_h2, masked_or_magic);
    x = x - magic;
    x = __builtin_elementwise_fma(x, sc, bi);
    return __builtin_bit_cast(uint32_t, x);
}
// position p of an aligned run of 8 codes of a K row in LDS holds code K_PERM<BITS>(p) of the run: the order in
// which the masked words above yield their pairs; the query operands are permuted the same way
template <int BITS> __device__ __forceinline__ constexpr int k_perm(int p) {
    return BITS == 4 ? ((p >> 1) + 4 * (p & 1)) : ((p & 4) | ((p & 2) >> 1) | ((p & 1) << 1));
}

// BITS 0: full precision (DT 0 fp16 / 1 bf16); 4 / 8: quantized (scales of dtype DT).
// QT = 16-row query tiles per wavefront (2: 128 rows per workgroup, 1: 64 rows, chosen by
// the launcher so that the grid fills the chip).  MM: 0 no mask, 1 index-only mask
// (causal / window, no memory access in the loop), 2 array mask.
// DK and DV are the head sizes of keys / queries and of values / outputs (192 and 128 for the multi-head latent
// attention models, equal otherwise).
template <int BITS, int DK, int DV, int DT, bool IDENT, int QT, int MM>
__global__ void __launch_bounds__(256, 2)
prefill_kernel(AttendArgs a, int nsplit) {
    static_assert(BITS == 4 || BITS == 8, "quantized caches only");
    constexpr int BM = 64 * QT;
    constexpr int KS = DK + 8;   // halves per K row in LDS (padded against bank conflicts)
    constexpr int VS = BN + 4;   // halves per V^T row in LDS
    constexpr int S = DK / 32;   // contraction steps over the head dim
    constexpr int NDT = DV / 16; // 16-row tiles of out^T
    __shared__ __attribute__((aligned(16))) _Float16 Ks[BN * KS];
    __shared__ __attribute__((aligned(16))) _Float16 Vs[DV * VS];
    __shared__ int rows_s[BN];
    __shared__ int tile_full_s;
    __shared__ __attribute__((aligned(16))) _Float16 sb_s[(DV / 32) * 2 * BN];  // V scales and biases: [group][scale, bias][token]

    const Store &st = a.st;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, jj = lane >> 4;
    // Linear workgroup ids go to the 8 XCDs round-robin and each XCD has its own L2: all query
    // blocks of one (batch, kv-head) pair get ids of the same residue, so the pair's K/V tiles
    // stay hot in one L2.
    const int r = a.Hq / a.Hkv;
    const int R = r * a.L;
    const int nblk = (R + BM - 1) / BM;
    int blk_x, bh, split;
    {
        const int id = blockIdx.x;
        const int BH = a.st.BH;
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
    // Under a causal or window mask the later query blocks see more keys: they get the lower workgroup ids,
    // which the hardware starts first, so that the launch does not end on its longest blocks.
    if (MM == 1) blk_x = nblk - 1 - blk_x;
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int row0 = blk_x * BM + wave * 16 * QT;  // first query row of this wavefront
    const float fill = finfo_min_dt(DT);
    const SymMask sym = sym_mask_init(a.mask, b, a.L, a.T);

    // ---- query operands: B of S^T = K . Q^T; lane (n, jj) holds q[row][32 s + 8 jj ..] ----
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
        // rows past R read row (rep 0, l 0), which is in bounds, and are zeroed: no branch around the
        // loads, which are one 16-byte piece per contraction step, all in flight together
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
                float v0 = DT == 0 ? (float)__builtin_bit_cast(_Float16, (uint16_t)pair) : __uint_as_float(pair << 16);
                float v1 = DT == 0 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(pair >> 16)) : __uint_as_float(pair & 0xffff0000u);
                qv[2 * w] = q_ok[qt] ? round_dt<DT>(v0 * a.scale) : 0.f;  // the reference rounds q * scale to T
                qv[2 * w + 1] = q_ok[qt] ? round_dt<DT>(v1 * a.scale) : 0.f;
            }
            // (the contraction order inside a run of 8 follows the staged K rows)
#pragma unroll
            for (int w = 0; w < 4; ++w) qop[qt][s].u[w] = h2_bits(qv[k_perm<BITS>(2 * w)], qv[k_perm<BITS>(2 * w + 1)]);
        }
    }

    f4 oacc[QT][NDT];
    float m_run[QT], l_run[QT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        m_run[qt] = -INFINITY;
        l_run[qt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) oacc[qt][dt] = f4{0.f, 0.f, 0.f, 0.f};
    }

    // ---- visible slot range for symbolic masks (only when slots are presented rows) -------
    int tile_lo = 0, tile_hi = (a.slots + BN - 1) / BN;
    if (IDENT) {
        const int i_first = blk_x * BM, i_last = min(R, i_first + BM) - 1;
        const bool spans = (i_first / a.L) != (i_last / a.L);
        const int l_min = spans ? 0 : i_first % a.L, l_max = spans ? a.L - 1 : i_last % a.L;
        if (a.mask.mode == KVHIP_MASK_CAUSAL) {
            tile_hi = min(tile_hi, (a.T - a.L + l_max) / BN + 1);
        } else if (a.mask.mode == KVHIP_MASK_WINDOW) {
            tile_hi = min(tile_hi, (a.mask.offset + l_max) / BN + 1);
            if (a.mask.window > 0) tile_lo = max(0, (a.mask.offset + l_min - a.mask.window + 1) / BN);
        }
        tile_hi = min(tile_hi, (a.T + BN - 1) / BN);
        if (sym_mask_some_row_empty(sym)) {  // a fully masked row averages over every key
            tile_lo = 0;
            tile_hi = (a.slots + BN - 1) / BN;
        }
    }

    // presented rows [keep_lo, keep_hi] are seen by every query row of this workgroup: a key
    // tile made only of such rows needs no per-element test (flag set while staging)
    int keep_lo = 0, keep_hi = -1;
    if (MM != 2) {
        keep_hi = a.T - 1;
        if (MM == 1) {
            const int i_first = blk_x * BM, i_last = min(R, i_first + BM) - 1;
            const bool spans = (i_first / a.L) != (i_last / a.L);
            const int l_min = spans ? 0 : i_first % a.L, l_max = spans ? a.L - 1 : i_last % a.L;
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

    // ---- optional split of the key range (small grids): each part leaves an
    // unnormalised partial per query row, merged by the decode path's combine kernel
    if (nsplit > 1) {
        const int span = (tile_hi - tile_lo + nsplit - 1) / nsplit;
        tile_lo = tile_lo + split * span;
        tile_hi = min(tile_hi, tile_lo + span);
    }

    // ---- staging: a tile is fetched from global memory into registers one iteration ahead
    // (in flight while the current tile is contracted), then converted and written to LDS.
    constexpr int BB = BITS;
    // K: KT threads per token row, CPT codes each: 8 threads where that gives whole packed words
    // (head sizes 64, 128 and 256), 4 otherwise (96 / 192: 24 / 48 codes = whole words, which may
    // straddle two groups of 32)
    constexpr int KT = (DK == 64 || DK == 128 || DK == 256) ? 8 : 4;
    constexpr int CPT = DK / KT;
    constexpr int KQW = CPT * BB / 32;            // packed words per thread for K
    static_assert((CPT * BB) % 32 == 0, "a thread's K codes are whole packed words");
    constexpr int VQW = 16 * BB / 32;             // packed words per thread and column for V
    constexpr int VCOLS = (2 * DV + 255) / 256;    // (column, half) items per thread for V
    uint32_t kq[KQW], vq[VCOLS * VQW], ksb_raw = 0, ksb_raw_hi = 0;
    uint32_t vsb_raw[DV / 32];
    int row_reg = -1;
    const int kt = tid / KT, kpart = tid % KT;
    const bool k_on = KT == 8 || tid < BN * KT;   // with 4 threads per row the upper half has no K work

    PageCursor page_cur(st, min(tile_lo * BN, max(a.slots - 1, 0)));  // tiles of 32 slots: the entry is fetched once per eight tiles
    auto fetch = [&](int tile) {
        const int slot0 = tile * BN;
        if (tid < BN) {
            const int slot = slot0 + tid;
            int row;
            if (IDENT) row = slot;
            else row = slot < a.slots ? slot_to_row(a.runs, slot) : -1;
            row_reg = (row >= 0 && row < a.T) ? row : -1;
        }
        const PageEntry &pe = page_cur.at(st, slot0);
        const int in_page = slot0 & (PAGE - 1);
        const char *cell = pe.v + (size_t)bh * st.v_cell;
        if (k_on) {
            const uint32_t *w = reinterpret_cast<const uint32_t *>(pe.k + (size_t)bh * st.k_cell + (size_t)(in_page + kt) * st.k_row) + kpart * KQW;
#pragma unroll
            for (int e = 0; e < KQW; ++e) kq[e] = w[e];
            // 8 threads per row: the D/8 codes of this thread lie in one group (group sizes are >= 32 >= D/8);
            // 4 threads per row: in at most two, the first code's and the last code's
            const uint32_t *sbp = reinterpret_cast<const uint32_t *>(pe.ksb + (size_t)bh * st.ksb_cell + (size_t)(in_page + kt) * st.ksb_row);
            ksb_raw = sbp[(kpart * CPT) / st.gs];
            if constexpr (KT != 8) ksb_raw_hi = sbp[(kpart * CPT + CPT - 1) / st.gs];
        }
        if (tid < BN) {
            const uint32_t *sb = reinterpret_cast<const uint32_t *>(pe.vsb + (size_t)bh * st.vsb_cell + (size_t)(in_page + tid) * st.vsb_row);
#pragma unroll
            for (int gg = 0; gg < DV / 32; ++gg)
                if (gg < DV / st.gs) vsb_raw[gg] = sb[gg];
        }
        const int tbase = slot0 & 32;
#pragma unroll
        for (int ci = 0; ci < VCOLS; ++ci) {
            const int c = tid + 256 * ci;
            if (c < 2 * DV) {
                const int d = c >> 1, part = c & 1;
                const uint32_t *vw = reinterpret_cast<const uint32_t *>(cell + v_row_off(st, slot0, d)) + (tbase + part * 16) * BB / 32;
#pragma unroll
                for (int e = 0; e < VQW; ++e) vq[ci * VQW + e] = vw[e];
            }
        }
    
    };
    auto sb_pair = [&](uint32_t raw, float &sc, float &bi) {  // (scale, bias) of a 16-bit dtype
        if (DT == 0) {
            sc = (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
            bi = (float)__builtin_bit_cast(_Float16, (uint16_t)(raw >> 16));
        } else {
            sc = __uint_as_float(raw << 16);
            bi = __uint_as_float(raw & 0xffff0000u);
        }
    };
    auto stage_k = [&]() {  // K, row indices and (quantized) the V scale/bias table
        if (tid < BN) rows_s[tid] = row_reg;
        if (wave == 0) {
            const bool full = __all(lane >= BN || (row_reg >= keep_lo && row_reg <= keep_hi));
            if (lane == 0) tile_full_s = full;
        }
        constexpr int per = 32 / BB;
        const kv_h2 m1024 = kv_h2{(_Float16)1024.f, (_Float16)1024.f}, m64 = kv_h2{(_Float16)64.f, (_Float16)64.f};
        if (k_on) {
            float sc, bi, sc_hi = 0.f, bi_hi = 0.f;
            sb_pair(ksb_raw, sc, bi);
            [[maybe_unused]] int g_lo = 0;
            if constexpr (KT != 8) {
                sb_pair(ksb_raw_hi, sc_hi, bi_hi);
                g_lo = (kpart * CPT) / st.gs;
            }
            const kv_h2 s_lo = kv_h2{(_Float16)sc, (_Float16)sc}, b_lo = kv_h2{(_Float16)bi, (_Float16)bi};
            [[maybe_unused]] const kv_h2 s_hi = kv_h2{(_Float16)sc_hi, (_Float16)sc_hi}, b_hi = kv_h2{(_Float16)bi_hi, (_Float16)bi_hi};
            _Float16 *dst = Ks + kt * KS + kpart * CPT;
#pragma unroll
            for (int e = 0; e < KQW; ++e) {
                kv_h2 s_ = s_lo, b_ = b_lo;
                if constexpr (KT != 8) {  // a packed word lies in one group (32 is a multiple of the codes per word)
                    if ((kpart * CPT + e * per) / st.gs != g_lo) {
                        s_ = s_hi;
                        b_ = b_hi;
                    }
                }
                const uint32_t w = kq[e];
                if constexpr (BB == 4) {  // codes (0,4) (1,5) (2,6) (3,7) of the word's 8
                    u4 o;
                    o.x = deq_pair((w & 0x000f000fu) | 0x64006400u, m1024, s_, b_);
                    o.y = deq_pair((w & 0x00f000f0u) | 0x54005400u, m64, s_, b_);
                    o.z = deq_pair(((w >> 8) & 0x000f000fu) | 0x64006400u, m1024, s_, b_);
                    o.w = deq_pair(((w >> 8) & 0x00f000f0u) | 0x54005400u, m64, s_, b_);
                    *reinterpret_cast<u4 *>(dst + e * 8) = o;
                } else {  // codes (0,2) (1,3) of the word's 4
                    uint2 o;
                    o.x = deq_pair((w & 0x00ff00ffu) | 0x64006400u, m1024, s_, b_);
                    o.y = deq_pair(((w >> 8) & 0x00ff00ffu) | 0x64006400u, m1024, s_, b_);
                    *reinterpret_cast<uint2 *>(dst + e * 4) = o;
                }
            }
        }
        if (tid < BN) {
#pragma unroll
            for (int gg = 0; gg < DV / 32; ++gg)
                if (gg < DV / st.gs) {
                    float s2, b2;
                    sb_pair(vsb_raw[gg], s2, b2);
                    sb_s[(gg * 2) * BN + tid] = (_Float16)s2;
                    sb_s[(gg * 2 + 1) * BN + tid] = (_Float16)b2;
                }
        }
    
    };
    auto stage_v = [&]() {
        const kv_h2 m1024 = kv_h2{(_Float16)1024.f, (_Float16)1024.f}, m64 = kv_h2{(_Float16)64.f, (_Float16)64.f};
#pragma unroll
        for (int ci = 0; ci < VCOLS; ++ci) {
            const int c = tid + 256 * ci;
            if (c < 2 * DV) {
                const int d = c >> 1, part = c & 1;
                uint32_t *dst = reinterpret_cast<uint32_t *>(Vs + d * VS + part * 16);
                const int g = d / st.gs;
                // the 16 tokens' scales and biases, two tokens per word
                const u4 *sp = reinterpret_cast<const u4 *>(sb_s + (g * 2) * BN + part * 16);
                const u4 *bp = reinterpret_cast<const u4 *>(sb_s + (g * 2 + 1) * BN + part * 16);
                const u4 sA = sp[0], sB = sp[1], bA = bp[0], bB = bp[1];
                const uint32_t sw[8] = {sA.x, sA.y, sA.z, sA.w, sB.x, sB.y, sB.z, sB.w};
                const uint32_t bw[8] = {bA.x, bA.y, bA.z, bA.w, bB.x, bB.y, bB.z, bB.w};
                auto S2 = [&](int tp) { return __builtin_bit_cast(kv_h2, sw[tp]); };
                auto B2 = [&](int tp) { return __builtin_bit_cast(kv_h2, bw[tp]); };
                // a word of a V tile row yields its tokens two at a time in token order (V tile order)
                if constexpr (BB == 4) {
#pragma unroll
                    for (int e = 0; e < 2; ++e) {  // 8 tokens per word
                        const uint32_t w = vq[ci * VQW + e];
                        dst[4 * e] = deq_pair((w & 0x000f000fu) | 0x64006400u, m1024, S2(4 * e), B2(4 * e));
                        dst[4 * e + 1] = deq_pair((w & 0x00f000f0u) | 0x54005400u, m64, S2(4 * e + 1), B2(4 * e + 1));
                        dst[4 * e + 2] = deq_pair(((w >> 8) & 0x000f000fu) | 0x64006400u, m1024, S2(4 * e + 2), B2(4 * e + 2));
                        dst[4 * e + 3] = deq_pair(((w >> 8) & 0x00f000f0u) | 0x54005400u, m64, S2(4 * e + 3), B2(4 * e + 3));
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {  // 4 tokens per word
                        const uint32_t w = vq[ci * VQW + e];
                        dst[2 * e] = deq_pair((w & 0x00ff00ffu) | 0x64006400u, m1024, S2(2 * e), B2(2 * e));
                        dst[2 * e + 1] = deq_pair(((w >> 8) & 0x00ff00ffu) | 0x64006400u, m1024, S2(2 * e + 1), B2(2 * e + 1));
                    }
                }
            }
        }
    };

    if (tile_lo < tile_hi) fetch(tile_lo);
    for (int tile = tile_lo; tile < tile_hi; ++tile) {
        if (tile > tile_lo) __syncthreads();  // everyone is done reading the previous tile
        stage_k();
        __syncthreads();  // the V dequantisation reads the scale/bias table
        stage_v();
        __syncthreads();
        if (tile + 1 < tile_hi) fetch(tile + 1);

        // ---- S^T = K . Q^T: acc[qt][mt] rows = tokens 16 mt + 4 jj + i, column = query n -----
        f4 sacc[QT][2];
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) sacc[qt][mt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            Op8 ka[S];  // all K operands of this 16-token half first, then the MFMAs back to back
#pragma unroll
            for (int s = 0; s < S; ++s)
                ka[s].v = *reinterpret_cast<const uint4 *>(Ks + (16 * mt + n) * KS + 32 * s + 8 * jj);
#pragma unroll
            for (int s = 0; s < S; ++s)
#pragma unroll
                for (int qt = 0; qt < QT; ++qt)
                    sacc[qt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[s].h, qop[qt][s].h, sacc[qt][mt], 0, 0, 0);
        }
        int trow[2][4];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) trow[mt][i] = rows_s[16 * mt + 4 * jj + i];
        const bool tile_full = tile_full_s != 0;

        // ---- online softmax per query column; P^T stays in place as the PV B operand ------
        // Tiles every query row of the workgroup sees completely (all slots live rows, inside
        // the mask for every row) skip the per-element tests.
        // a boolean array mask is read four keys at a time where this lane's four rows are consecutive
        [[maybe_unused]] bool vec_ok[2] = {false, false};
        if constexpr (MM == 2) {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                vec_ok[mt] = a.mask.dtype == KVHIP_BOOL && trow[mt][0] >= 0 && trow[mt][3] == trow[mt][0] + 3 &&
                             trow[mt][1] == trow[mt][0] + 1 && trow[mt][2] == trow[mt][0] + 2;
        }
        Op8 pb[QT];
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            [[maybe_unused]] uint32_t mword[2] = {0u, 0u};
            if constexpr (MM == 2) {
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
                    if (vec_ok[mt] && q_ok[qt]) {
                        uint32_t w[1];
                        mask_bool_words<1>(a.mask, b, q_h[qt], q_l[qt], trow[mt][0], w);
                        mword[mt] = w[0];
                    }
            }
            float sc[2][4];
            float tmax = -INFINITY;
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float s_ = round_dt<DT>(sacc[qt][mt][i]);
                    if (MM == 2 || !tile_full) {  // workgroup-uniform
                        const int row = trow[mt][i];
                        if (row >= 0 && q_ok[qt]) {
                            if constexpr (MM == 1) {
                                if (!sym_mask_keep(sym, q_l[qt], row)) s_ = fill;
                            } else if constexpr (MM == 2) {
                                if (vec_ok[mt]) {
                                    if (((mword[mt] >> (8 * i)) & 0xffu) == 0u) s_ = fill;
                                } else {
                                    float add;
                                    const bool keep = mask_keep(a.mask, b, q_h[qt], q_l[qt], row, a.L, a.T, add);
                                    if (!keep) s_ = fill;
                                    else if (a.mask.dtype != KVHIP_BOOL) s_ = round_dt<DT>(s_ + add);
                                }
                            }
                        } else {
                            s_ = -INFINITY;
                        }
                    }
                    sc[mt][i] = s_;
                    tmax = fmaxf(tmax, s_);
                }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
            // m_run is a reference value rather than the exact running maximum: it is raised (to the
            // maximum seen) only when a score exceeds it by more than RAISE, so p stays below
            // e^RAISE = 256 and the accumulators are rescaled a handful of times per query
            if (__any(tmax > m_run[qt] + RAISE)) {
                const float mn = fmaxf(m_run[qt], tmax);
                const float alpha = (mn == -INFINITY) ? 1.f : exp2_fast((m_run[qt] - mn) * LOG2E);
                m_run[qt] = mn;
                l_run[qt] *= alpha;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) oacc[qt][dt][i] *= alpha;
            }
            const float mu = (m_run[qt] == -INFINITY) ? 0.f : m_run[qt];
            float psum = 0.f;
            float p[2][4];
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    p[mt][i] = exp2_fast((sc[mt][i] - mu) * LOG2E);  // exp2(-inf) = 0 for excluded keys
                    psum += p[mt][i];
                }
            l_run[qt] += psum;
            pb[qt].u[0] = h2_bits(p[0][0], p[0][1]);
            pb[qt].u[1] = h2_bits(p[0][2], p[0][3]);
            pb[qt].u[2] = h2_bits(p[1][0], p[1][1]);
            pb[qt].u[3] = h2_bits(p[1][2], p[1][3]);
        }

        // ---- out^T += V^T . P^T: A = V^T rows (tokens 4jj..4jj+3 and 16+4jj..) from LDS -------
#pragma unroll
        for (int d0 = 0; d0 < NDT; d0 += 4) {
            Op8 va[4];  // four V^T operands per batch of LDS reads
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const _Float16 *vrow = Vs + (16 * (d0 + x) + n) * VS;
                va[x].d2[0] = *reinterpret_cast<const uint2 *>(vrow + 4 * jj);
                va[x].d2[1] = *reinterpret_cast<const uint2 *>(vrow + 16 + 4 * jj);
            }
#pragma unroll
            for (int x = 0; x < 4; ++x)
#pragma unroll
                for (int qt = 0; qt < QT; ++qt)
                    oacc[qt][d0 + x] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[x].h, pb[qt].h, oacc[qt][d0 + x], 0, 0, 0);
        }
    }

    // ---- normalise and store: lane (n, jj) holds out[q = n][d = 16 dt + 4 jj + i] ------------
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        float l = l_run[qt];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        if (!q_ok[qt]) continue;
        if (nsplit > 1) {
            const int i = row0 + 16 * qt + n;
            float *part = a.workspace + (((size_t)bh * nsplit + split) * R + i) * (DV + 2);
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
                *reinterpret_cast<f4 *>(part + 16 * dt + 4 * jj) = oacc[qt][dt];
            if (jj == 0) {
                part[DV] = m_run[qt];
                part[DV + 1] = l;
            }
            continue;
        }
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        const size_t ooff = ((size_t)(b * a.Hq + q_h[qt]) * a.L + q_l[qt]) * DV;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) Elem<DT>::store(a.out, ooff + 16 * dt + 4 * jj + i, oacc[qt][dt][i] * inv);
    }
}

}  // namespace

bool attend_prefill_supported(const AttendArgs &a) {
    const Store &s = a.st;
    if (s.dtype != KVHIP_F16 && s.dtype != KVHIP_BF16) return false;
    // keys of 192 with values of 128 (the multi-head latent attention models): full precision, or 4- / 8-bit codes
    // in groups of 32 or 64 (the sizes that divide both)
    if (s.Dk == 192 && s.Dv == 128 && (s.bits == 0 || ((s.bits == 4 || s.bits == 8) && (s.gs == 32 || s.gs == 64)))) return true;
    if (s.Dk != s.Dv) return false;
    // head sizes 80 (full precision only) and 96: every row count (no decode kernel is built for them)
    if (s.Dk != 64 && s.Dk != 128 && s.Dk != 256 && s.Dk != 96 && !(s.Dk == 80 && s.bits == 0)) return false;
    if (s.bits != 0 && s.gs < 32) return false;
    if (s.bits != 0 && s.Dk != 96) return attend_prefill_q_supported(a);  // the pipelined tile (every code width): slots in presented order
    if (s.bits != 0 && s.bits != 4 && s.bits != 8) return false;
    return true;  // 16 rows or fewer come here only when the decode kernels do not take the shape
}

// 128 query rows per workgroup reuse each staged tile twice as often as 64; 64 rows are
// used when that would leave the grid too small to fill 256 CUs twice over.
static bool prefill_wide(const AttendArgs &a) {
    const int R = (a.Hq / a.Hkv) * a.L;
    static const int forced = measure_knob("KVHIP_PREFILL_WIDE", -1);  // (timing builds only)
    if (forced >= 0) return forced != 0 && a.st.Dk <= 128;
    return (size_t)((R + 127) / 128) * a.st.BH >= 512 && a.st.Dk <= 128;
}

// Query rows per workgroup.  The pipelined tile for quantized caches (kvhip_attend_prefill_q.hip) takes 256 rows
// on 8 wavefronts at head size 128, one workgroup per CU, whenever that still gives every CU a workgroup: four
// times as many rows share each converted tile (B1, 2048 x 8192, 4 bits: 552 against 446 TFLOP/s; a square causal
// 4096 x 4096, which would leave half the CUs empty, stays on 64 rows: 480 against 380).  Otherwise 128 or 64 rows
// on 4 wavefronts as above (quantized: 64).
static int prefill_block_rows(const AttendArgs &a) {
    const int R = (a.Hq / a.Hkv) * a.L;
    if (a.st.bits != 0 && attend_prefill_q_supported(a)) {
        static const int forced = measure_knob("KVHIP_PREFILL_ROWS", 0);  // (timing builds only)
        if (a.st.bits != 4 && a.st.bits != 8) return 64;
        if (forced > 0 && a.st.Dk == 128) return forced;
        // (head size 64 measured faster on 64 rows: 363 / 393 against 340 / 362 TFLOP/s at 8 / 4 bits, B4 2048 x 4096)
        return ((size_t)((R + 255) / 256) * a.st.BH >= 256 && a.st.Dk == 128) ? 256 : 64;
    }
    return prefill_wide(a) ? 128 : 64;
}

// Key-range parts per query block: only when the grid would leave most CUs without a
// second workgroup, and only while the partials stay small.
static int prefill_splits(const AttendArgs &a) {
    const int R = (a.Hq / a.Hkv) * a.L;
    const int bm = prefill_block_rows(a);
    if (bm == 256) return 1;  // (chosen only when the grid fills the chip)
    const size_t wgs = (size_t)((R + bm - 1) / bm) * a.st.BH;
    // as many workgroups as are resident at once: three per CU, two at D = 256 (LDS) -- a part more
    // than that starts a second round that leaves half the CUs idle
    static const int forced = measure_knob("KVHIP_PREFILL_TARGET", 0);  // (timing builds only)
    const int target = forced > 0 ? forced : (a.st.Dk >= 256 ? 512 : 768);
    int n = (int)(target / (wgs ? wgs : 1));
    const int tiles = (a.slots + BN - 1) / BN;
    if (n > tiles / 8) n = tiles / 8;
    if (n > 8) n = 8;
    if (n < 2) return 1;
    const size_t per_part = (size_t)a.st.BH * R * (a.st.Dv + 2) * sizeof(float);
    if (per_part * n > ((size_t)256 << 20)) return 1;
    // a caller with a fixed amount of scratch: fewer parts until they fit (one part has no partials)
    while (a.workspace_cap && n > 1 && per_part * n > a.workspace_cap) --n;
    return n;
}

size_t attend_prefill_workspace(const AttendArgs &a) {
    const int n = prefill_splits(a);
    if (n <= 1) return 0;
    return (size_t)a.st.BH * n * (a.Hq / a.Hkv) * a.L * (a.st.Dv + 2) * sizeof(float);
}

hipError_t launch_attend_prefill(const AttendArgs &a, hipStream_t s) {
    const Store &st = a.st;
    const int R = (a.Hq / a.Hkv) * a.L;
    // 128 query rows per workgroup reuse each staged tile twice as often; 64 rows are used
    // when that would leave the grid too small to fill 256 CUs twice over
    const int bm = prefill_block_rows(a);
    const bool wide = bm == 128;
    const int nsplit = prefill_splits(a);
    dim3 grid((unsigned)((R + bm - 1) / bm) * st.BH * nsplit), block(256);  // linear: the kernel maps ids to tiles
    const bool ident = a.runs.n == 1 && a.runs.row0[0] == 0 && a.runs.phys0[0] == 0;
    const int mm = a.mask.mode == KVHIP_MASK_NONE ? 0 : (a.mask.mode == KVHIP_MASK_ARRAY ? 2 : 1);
#define PF_M(BITS, D, DT, QT, MM)                                                                         \
    do {                                                                                                  \
        profile_mark(s, true);                                                                            \
        if (ident) hipLaunchKernelGGL((prefill_kernel<BITS, D, D, DT, true, QT, MM>), grid, block, 0, s, a, nsplit); \
        else hipLaunchKernelGGL((prefill_kernel<BITS, D, D, DT, false, QT, MM>), grid, block, 0, s, a, nsplit);      \
        profile_mark(s, false);                                                                           \
    } while (0)
#define PF(BITS, D, DT, QT)                      \
    do {                                         \
        if (mm == 0) PF_M(BITS, D, DT, QT, 0);   \
        else if (mm == 1) PF_M(BITS, D, DT, QT, 1); \
        else PF_M(BITS, D, DT, QT, 2);           \
    } while (0)
#define PF_QT(BITS, D, DT)                       \
    do {                                         \
        if (wide) PF(BITS, D, DT, 2);            \
        else PF(BITS, D, DT, 1);                 \
    } while (0)
#define PF_DT(BITS, D)                           \
    do {                                         \
        if (st.dtype == KVHIP_F16) PF_QT(BITS, D, 0); \
        else PF_QT(BITS, D, 1);                  \
    } while (0)
#define PF_MLA(BITS, DT)                                                                                   \
    do {                                                                                                  \
        profile_mark(s, true);                                                                            \
        if (mm == 0) {                                                                                    \
            if (ident) hipLaunchKernelGGL((prefill_kernel<BITS, 192, 128, DT, true, 1, 0>), grid, block, 0, s, a, nsplit);  \
            else hipLaunchKernelGGL((prefill_kernel<BITS, 192, 128, DT, false, 1, 0>), grid, block, 0, s, a, nsplit);       \
        } else if (mm == 1) {                                                                             \
            if (ident) hipLaunchKernelGGL((prefill_kernel<BITS, 192, 128, DT, true, 1, 1>), grid, block, 0, s, a, nsplit);  \
            else hipLaunchKernelGGL((prefill_kernel<BITS, 192, 128, DT, false, 1, 1>), grid, block, 0, s, a, nsplit);       \
        } else {                                                                                          \
            if (ident) hipLaunchKernelGGL((prefill_kernel<BITS, 192, 128, DT, true, 1, 2>), grid, block, 0, s, a, nsplit);  \
            else hipLaunchKernelGGL((prefill_kernel<BITS, 192, 128, DT, false, 1, 2>), grid, block, 0, s, a, nsplit);       \
        }                                                                                                 \
        profile_mark(s, false);                                                                           \
    } while (0)
#define PF_D(BITS)                                    \
    do {                                              \
        if (st.Dk == 192) { /* keys 192 / values 128: 64 query rows per workgroup */ \
            if (st.dtype == KVHIP_F16) PF_MLA(BITS, 0); else PF_MLA(BITS, 1);        \
        } else if (st.Dk == 96) PF_DT(BITS, 96);      \
        else return hipErrorInvalidValue; /* 64 / 128 / 256 are served above */ \
    } while (0)
    if (st.bits != 0 && attend_prefill_q_supported(a)) {
        // head sizes 64 / 128 / 256: the pipelined tile of kvhip_attend_prefill_q.hip
        profile_mark(s, true);
        hipError_t e = launch_attend_prefill_q(a, nsplit, bm, s);
        profile_mark(s, false);
        if (e != hipSuccess) return e;
    } else if (st.bits == 4) PF_D(4);
    else if (st.bits == 8) PF_D(8);
    else {
        // full-precision caches have their own double-buffered kernel
        profile_mark(s, true);
        hipError_t e = launch_attend_prefill_fp(a, nsplit, wide, s);
        profile_mark(s, false);
        if (e != hipSuccess) return e;
    }
#undef PF_D
#undef PF_MLA
#undef PF_DT
#undef PF_QT
#undef PF
#undef PF_M
    if (nsplit > 1) {
        hipError_t e = launch_combine(a, nsplit, R, s);
        if (e != hipSuccess) return e;
    }
    return hipGetLastError();
}

}  // namespace kvhip
