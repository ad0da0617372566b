// Chunked-prefill attention for full-precision caches (fp16 / bf16) on the matrix cores
// (gfx950, v_mfma_f32_16x16x32_f16 / _bf16).
//
// One workgroup (4 wavefronts) owns 64 (QT = 1) or 128 (QT = 2) query rows of one
// (batch, kv-head) pair and walks the cached keys in tiles of 32 slots:
//   S^T   = K . Q^T      A = K rows from LDS in the cache's own dtype (no conversion),
//                        B = query rows held in registers
//   out^T += V^T . P^T   A = V^T rows from LDS as fp16 (bf16 is converted while staging),
//                        B = the fp16 probabilities exactly where the S^T accumulators left
//                        them, so P never moves between lanes
// K/V tiles are double-buffered in LDS: while a tile is contracted, the next one (already in
// registers) is written to the other buffer and the one after that is requested from global
// memory, with a single barrier per tile.  Global reads and LDS writes of a tile are
// chunk-interleaved over the 256 threads (consecutive lanes, consecutive 16 bytes), LDS rows
// are padded so that both the writes and the operand reads are bank-conflict free.
// The online softmax rescales the accumulators only when a row maximum rises, and key tiles
// that every query row of the workgroup sees completely skip all mask tests.
#include "kvhip_mask.hpp"

#ifndef KVHIP_PREFILL_LM
#define KVHIP_PREFILL_LM 1
#endif
#ifndef KVHIP_PREFILL_BF16_P
#define KVHIP_PREFILL_BF16_P 1
#endif

namespace kvhip {

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) uint32_t LDS_U32;

// 16 bytes per lane from global memory straight into LDS: lane i's land at `lds_wave_base` + 16 i
// (the base is the same for the whole wavefront).  Written as assembly, with the waits for it placed
// by hand (s_waitcnt vmcnt): the compiler's own bookkeeping of such loads makes every LDS read that
// follows one wait for all vector-memory operations in flight, register loads included, wherever it
// cannot prove on every path which buffer the load fills.  Its waits for its own loads stay correct:
// vector-memory operations complete in order, so an operation it does not count only makes a wait
// stricter.
// INVARIANT for anyone who edits this kernel: (1) every wavefront of the workgroup issues the same
// number of these loads per step (the repeated tail chunks at D = 80 / 96 exist for that), because
// the hand-placed `s_waitcnt vmcnt(N)` count them; (2) a step ends with vmcnt(0) and a barrier before
// any wavefront reads the buffer the loads fill; (3) vector-memory operations of one wavefront
// complete in order on this hardware -- the compiler's own waits for register loads rely on that
// when an uncounted LDS load sits between them.  A new load inside the loop, or a different order of
// `stage` / `fetch` / `dma`, has to keep all three.
__device__ __forceinline__ void load_to_lds(const void *src, const void *lds_wave_base) {
    // (the low half of a flat address inside the LDS aperture is the LDS address itself)
    const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds_wave_base);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(base) : "memory", "m0");
}
union Op8 {
    h8 h;
    b8 b;
    u4 v;
};

constexpr int BN = 32;  // key slots per tile
constexpr float LOG2E = 1.4426950408889634f;
constexpr float RAISE = 8.f;  // log2 units

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ uint32_t rn_h2(float lo, float hi) {  // round to nearest even
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
}
// two non-negative finite floats -> two bf16 (round to nearest even) in one dword
__device__ __forceinline__ uint32_t rn_bf2(float lo, float hi) {
    const uint32_t a = __float_as_uint(lo), b = __float_as_uint(hi);
    return ((a + 0x7fffu + ((a >> 16) & 1u)) >> 16) | ((b + 0x7fffu + ((b >> 16) & 1u)) & 0xffff0000u);
}
// the probabilities of one lane as the PV operand: fp16, or bf16 for bf16 caches on the direct path
template <bool BF> __device__ __forceinline__ u4 pack_p(const float (&p)[2][4]) {
    if constexpr (BF) return u4{rn_bf2(p[0][0], p[0][1]), rn_bf2(p[0][2], p[0][3]), rn_bf2(p[1][0], p[1][1]), rn_bf2(p[1][2], p[1][3])};
    else return u4{rn_h2(p[0][0], p[0][1]), rn_h2(p[0][2], p[0][3]), rn_h2(p[1][0], p[1][1]), rn_h2(p[1][2], p[1][3])};
}
// two bf16 (one dword) -> two fp16, exact for every bf16 inside the fp16 range
__device__ __forceinline__ uint32_t bf2_to_h2(uint32_t w) {
    return rn_h2(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u));
}

__device__ __forceinline__ int st_BH(const AttendArgs &a) { return a.st.BH; }

template <int DT> __device__ __forceinline__ f4 mfma_qk(const Op8 &a, const Op8 &b, f4 c) {
    if constexpr (DT == 0) return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
}

// D = 256 runs 64 query rows per workgroup only: 128 rows need the accumulator registers of
// a whole SIMD lane (one wavefront per SIMD), which measured slower (0.34 ms against 0.29 ms
// for a 512 x 4607 chunk at B4, 8 query heads).
template <int D, int DT, bool IDENT, int QT, int MM>
__global__ void __launch_bounds__(256, 2)
prefill_fp_kernel(AttendArgs a, int nsplit) {
    constexpr int BM = 64 * QT;
    constexpr int VS = BN + 4;    // halves per V^T row in LDS: 18 dwords, so the 16 rows an operand
                                  // read touches fall in distinct banks
    constexpr int S = (D + 31) / 32;  // contraction steps over the head dim (the last one partly zero at D = 80)
    constexpr int NDT = D / 16;   // 16-row tiles of out^T
    constexpr int NC = (D + 63) / 64;  // rounds of 256 16-byte chunks, for K and for V
    constexpr int CH = 4 * D;          // 16-byte chunks of a tile's K (and of its V); a multiple of 64
    static_assert(D % 16 == 0, "out^T is built from 16-row tiles");
    // A head size that is not a multiple of 32 (80): the last contraction step reads K chunks past the
    // row -- the unused tail that the repeated loads fill with finite values -- against query
    // operands that are zero there.
    static_assert(4 * S * BN <= ((D + 63) / 64) * 256, "the padded contraction stays inside the staged buffer");
    // K tiles move from global memory straight into LDS (no registers, no LDS store instructions):
    // two buffers, each the tile's 16-byte chunks in page order, [8-element chunk][token], the other
    // one filled while this one is contracted.  fp16 caches move V the same way, [8-token
    // chunk][column]; bf16 V is staged through registers (converted to fp16 on the way) into two
    // padded buffers of V^T.
    // bf16 caches keep V as bf16 too: the probabilities are then rounded to bf16 for the PV matrix-core
    // instruction (the reference's softmax output is an array of the cache's dtype as well), so that V
    // needs no conversion and takes the direct path.  KVHIP_PREFILL_BF16_P = 0 brings back fp16
    // probabilities with V converted to fp16 while it is staged through registers.
    constexpr bool VDMA = DT == 0 || KVHIP_PREFILL_BF16_P;
    constexpr int NB = 2;
    // (one array per buffer, K then V, selected by constants after inlining: the compiler follows
    // loads into LDS per variable, and a read of one buffer then need not wait for the loads in
    // flight into the other)
    // 16-bit elements reserved for a tile's K (and for its V): whole rounds of 256 chunks.  With a head
    // size that is not a multiple of 64 (80, 96) the last round is partly empty: its wavefronts past the
    // tile's last chunk repeat that chunk into the unused tail, so that every wavefront issues the same
    // number of loads and the hand-placed waits below count alike in all of them.
    constexpr int KSZ = NC * 256 * 8;
    __shared__ __attribute__((aligned(16))) uint16_t KV0[VDMA ? 2 * KSZ : KSZ], KV1[VDMA ? 2 * KSZ : KSZ];
    __shared__ __attribute__((aligned(16))) _Float16 Vpad[2][VDMA ? 8 : D * VS];
    auto Ks = [&](int buf) __attribute__((always_inline)) -> uint16_t * { return buf == 0 ? KV0 : KV1; };
    auto Vs = [&](int buf) __attribute__((always_inline)) -> _Float16 * {
        if constexpr (VDMA) return reinterpret_cast<_Float16 *>(buf == 0 ? KV0 : KV1) + KSZ;
        else return Vpad[buf];
    };
    __shared__ int rows_s[NB][BN];
    __shared__ int full_s[NB];

    const Store &st = a.st;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, jj = lane >> 4;
    // Workgroups go to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  All
    // query blocks of one (batch, kv-head) pair re-read that pair's K and V, so they are given
    // ids of the same residue: a pair's tiles then stay hot in one L2 instead of missing in all.
    const int r = a.Hq / a.Hkv;
    const int R = r * a.L;
    const int nblk = (R + BM - 1) / BM;
    int blk_x, bh, split;
    {
        const int id = blockIdx.x;
        const int BH = st_BH(a);
        if ((BH & 7) == 0) {
            const int xcd = id & 7, j = id >> 3;
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
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int row0 = blk_x * BM + wave * 16 * QT;  // first query row of this wavefront
    const SymMask sym = sym_mask_init(a.mask, b, a.L, a.T);
    // Fast softmax (fp16 caches up to D = 128; D = 256 has no registers to spare, and bf16 keeps its
    // float32 denominators): scores enter as exp2(s * sl2 - m) with sl2 >= 0 -- a negative scale
    // flips the sign of the query operands instead (exact), a zero one becomes a vanishing positive
    // factor -- so that the maximum can be taken on the raw scores and the scale folded into one
    // multiply-add; the denominators ride on the matrix cores (lacc = ones . P^T sums the same
    // rounded probabilities the numerator uses; all 16 rows of the block hold the same sums).
    constexpr bool LM = D <= 128 && DT == 0 && KVHIP_PREFILL_LM;
    const bool flip = LM && a.scale < 0.f;
    const float sl2 = LM ? fmaxf(fabsf(a.scale) * LOG2E, 1e-30f) : a.scale * LOG2E;

    // ---- query operands: B of S^T = K . Q^T; lane (n, jj) holds q[row][32 s + 8 jj ..] raw ----
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
        const u4 *qp = reinterpret_cast<const u4 *>(
            reinterpret_cast<const uint16_t *>(a.q) + ((size_t)(b * a.Hq + q_h[qt]) * a.L + q_l[qt]) * D + 8 * jj);
#pragma unroll
        for (int s = 0; s < S; ++s) {
            u4 w = (q_ok[qt] && (D % 32 == 0 || 32 * s + 8 * jj < D)) ? qp[4 * s] : u4{0, 0, 0, 0};
            if (flip) w ^= u4{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
            qop[qt][s].v = w;
        }
    }

    f4 oacc[QT][NDT];
    float m_run[QT], l_run[QT];
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
    int tile_lo = 0, tile_hi = (a.slots + BN - 1) / BN;
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
        if (IDENT) {  // slots are presented rows: tiles outside a symbolic mask are skipped
            if (a.mask.mode == KVHIP_MASK_CAUSAL) {
                tile_hi = min(tile_hi, (a.T - a.L + l_max) / BN + 1);
            } else if (a.mask.mode == KVHIP_MASK_WINDOW) {
                tile_hi = min(tile_hi, (a.mask.offset + l_max) / BN + 1);
                if (a.mask.window > 0) tile_lo = max(0, (a.mask.offset + l_min - a.mask.window + 1) / BN);
            }
            tile_hi = min(tile_hi, (a.T + BN - 1) / BN);
        }
    }
    // optional split of the key range (small grids): each part leaves an
    // unnormalised partial per query row, merged by the decode path's combine kernel
    if (nsplit > 1) {
        const int span = (tile_hi - tile_lo + nsplit - 1) / nsplit;
        tile_lo = tile_lo + split * span;
        tile_hi = min(tile_hi, tile_lo + span);
    }

    // ---- staging ------------------------------------------------------------------------
    // chunk c = e * 256 + tid.  K: slot c % 32 of the tile, 8-element chunk c / 32.  V: column
    // c % D, 8-token chunk c / D of the 32 tokens of this tile.
    // V through registers: a tile's V is requested one iteration before it is written to LDS and two
    // before it is contracted.
    constexpr int LEAD = 2;
    struct Stg {
        u4 v[NC];
    };
    Stg setA;
    // tiles of 32 slots: the page-table entry is fetched once per eight tiles
    PageCursor page_fetch(st, min(tile_lo * BN, max(a.slots - 1, 0))), page_dma = page_fetch;
    [[maybe_unused]] auto fetch = [&](int tile, Stg &g) __attribute__((always_inline)) {
        const int slot0 = tile * BN;
        const char *vbase = page_fetch.at(st, slot0).v + (size_t)bh * st.v_cell + vfp_off(st, slot0, 0);
#pragma unroll
        for (int e = 0; e < NC; ++e) {
            const int c = min(e * 256 + tid, CH - 1);
            g.v[e] = *reinterpret_cast<const u4 *>(vbase + (size_t)(c / D) * (D * 16) + (c % D) * 16);
        }
    };
    [[maybe_unused]] auto stage = [&](int buf, const Stg &g) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < NC; ++e) {
            const int c = e * 256 + tid;
            if (c >= CH) continue;
            u4 v = g.v[e];
            if (DT == 1) v = u4{bf2_to_h2(v.x), bf2_to_h2(v.y), bf2_to_h2(v.z), bf2_to_h2(v.w)};
            u2 *vd = reinterpret_cast<u2 *>(&Vs(buf)[(c % D) * VS + (c / D) * 8]);  // rows are 8-byte aligned
            vd[0] = u2{v.x, v.y};
            vd[1] = u2{v.z, v.w};
        }
    };

    // direct global -> LDS: lane i of a wavefront's load lands at the wavefront's LDS base + 16 i, so
    // chunk c = e * 256 + tid goes to slot c of the buffer.  With V loaded the same way, K slot
    // (chunk cc, position pos) takes token 8 ((pos & 15) / 4) + 4 (pos / 16) + pos % 4, the order in
    // which the S^T accumulators of one lane cover the eight tokens of one V chunk (so K operand
    // reads are contiguous across lanes and P never moves), and V slots are the page's own order;
    // with V^T staged through registers K slots are the tokens in order.
    auto dma = [&](int tile, int buf) __attribute__((always_inline)) {
        const int slot0 = tile * BN;
        if (tid < BN) {
            const int pos = tid;
            const int slot = slot0 + (VDMA ? 8 * ((pos & 15) >> 2) + 4 * (pos >> 4) + (pos & 3) : pos);
            int row;
            if (IDENT) row = slot;
            else row = slot < a.slots ? slot_to_row(a.runs, slot) : -1;
            row = (row >= 0 && row < a.T) ? row : -1;
            rows_s[buf][tid] = row;  // the row of the token in K slot `tid`
            const bool full = __all(row >= keep_lo && row <= keep_hi);  // the first 32 lanes of wavefront 0
            if (tid == 0) full_s[buf] = full;
        }
        const PageEntry &pe = page_dma.at(st, slot0);
        const char *kbase = pe.k + (size_t)bh * st.k_cell + kfp_off(st, slot0, 0);
        const char *vbase = pe.v + (size_t)bh * st.v_cell + vfp_off(st, slot0, 0);
#pragma unroll
        for (int e = 0; e < NC; ++e) {
            const int c = min(e * 256 + tid, CH - 1);
            const int pos = c % BN;
            const int tok = VDMA ? 8 * ((pos & 15) >> 2) + 4 * (pos >> 4) + (pos & 3) : pos;
            const int cw = e * 256 + (tid & ~63);  // the wavefront's first slot
            load_to_lds(kbase + (size_t)(c / BN) * (TILE * 16) + tok * 16, &Ks(buf)[cw * 8]);
            if constexpr (VDMA) load_to_lds(vbase + (size_t)c * 16, &Vs(buf)[cw * 8]);
        }
    };
    // all but the `newer` most recent vector-memory operations of this wavefront have completed
    auto wait_older = [&](auto N) __attribute__((always_inline)) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(decltype(N)::value) : "memory");
    };

    // (fast softmax) raise query block qt's reference maximum to what the tile holds and rescale
    auto raise = [&](int qt, float tmax) __attribute__((always_inline)) {
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float mn = fmaxf(m_run[qt], tmax);
        const float alpha = (mn == -INFINITY) ? 1.f : exp2_fast(m_run[qt] - mn);
        m_run[qt] = mn;
#pragma unroll
        for (int i = 0; i < 4; ++i) lacc[LM ? qt : 0][i] *= alpha;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) oacc[qt][dt][i] *= alpha;
    };
    // one tile: `cur` is the LDS buffer that holds it, `g` the register set that holds the next one
    auto step = [&](int tile, int cur, Stg &g) __attribute__((always_inline)) {
        // The other buffers were last read in the previous step, which ended with a barrier.
        // V^T first (the tile fetched in the previous step; its registers are then free for the tile
        // after it), the K request last: the compiler's waits for those registers -- it does not
        // count the K request -- must not meet it.
        if constexpr (!VDMA) {
            if (tile + 1 < tile_hi) stage(cur ^ 1, g);
            if (tile + LEAD < tile_hi) fetch(tile + LEAD, g);
        }
        if (tile + 1 < tile_hi) dma(tile + 1, cur ^ 1);

        // ---- S^T = K . Q^T: acc[qt][mt] rows = tokens 16 mt + 4 jj + i, column = query n -----
        f4 sacc[QT][2];
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) sacc[qt][mt] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
            Op8 ka[S];
#pragma unroll
            for (int s = 0; s < S; ++s)
                ka[s].v = *reinterpret_cast<const u4 *>(&Ks(cur)[((4 * s + jj) * BN + 16 * mt + n) * 8]);
#pragma unroll
            for (int s = 0; s < S; ++s)
#pragma unroll
                for (int qt = 0; qt < QT; ++qt) sacc[qt][mt] = mfma_qk<DT>(ka[s], qop[qt][s], sacc[qt][mt]);
        }
        const bool tile_full = full_s[cur] != 0;
        int trow[2][4];
        if (MM == 2 || !tile_full) {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) trow[mt][i] = rows_s[cur][16 * mt + 4 * jj + i];  // by K slot
        }

        // a boolean array mask is read four keys at a time where this lane's four rows are consecutive
        [[maybe_unused]] bool vec_ok[2] = {false, false};
        if constexpr (MM == 2) {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                vec_ok[mt] = a.mask.dtype == KVHIP_BOOL && trow[mt][0] >= 0 && trow[mt][3] == trow[mt][0] + 3 &&
                             trow[mt][1] == trow[mt][0] + 1 && trow[mt][2] == trow[mt][0] + 2;
        }

        // ---- online softmax per query column; P^T stays in place as the PV B operand ------
        // Scores stay in the log2 domain: x = s * (scale * log2 e), p = exp2(x - m).  m is a reference
        // value rather than the exact running maximum: it is the same in the four lanes that share a
        // query and is raised (to the maximum seen) only when a score exceeds it by more than RAISE,
        // so p stays below 2^RAISE (exact in fp16, whose relative precision does not depend on
        // magnitude) and the accumulators are rescaled a handful of times per query, not on every
        // tile that happens to hold a new maximum.
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
            if constexpr (LM) {
                if (MM != 2 && tile_full) {
                    // every key of the tile counts for every query
                    float tmax = fmaxf(fmaxf(fmaxf(sacc[qt][0][0], sacc[qt][0][1]), fmaxf(sacc[qt][0][2], sacc[qt][0][3])),
                                       fmaxf(fmaxf(sacc[qt][1][0], sacc[qt][1][1]), fmaxf(sacc[qt][1][2], sacc[qt][1][3])));
                    tmax *= sl2;
                    if (__any(tmax > m_run[qt] + RAISE)) raise(qt, tmax);
                    const float mu = (m_run[qt] == -INFINITY) ? 0.f : m_run[qt];
                    float p[2][4];
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) p[mt][i] = exp2_fast(__builtin_fmaf(sacc[qt][mt][i], sl2, -mu));
                    pb[qt].v = u4{rn_h2(p[0][0], p[0][1]), rn_h2(p[0][2], p[0][3]), rn_h2(p[1][0], p[1][1]), rn_h2(p[1][2], p[1][3])};
                } else {
                    float x[2][4];
                    float tmax = -INFINITY;
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            float x_ = sacc[qt][mt][i] * sl2;
                            const int row = trow[mt][i];
                            if (row >= 0 && q_ok[qt]) {
                                if constexpr (MM == 1) {
                                    if (!sym_mask_keep(sym, q_l[qt], row)) x_ = -INFINITY;
                                } else if constexpr (MM == 2) {
                                    if (vec_ok[mt]) {
                                        if (((mword[mt] >> (8 * i)) & 0xffu) == 0u) x_ = -INFINITY;
                                    } else {
                                        float add;
                                        const bool keep = mask_keep(a.mask, b, q_h[qt], q_l[qt], row, a.L, a.T, add);
                                        x_ = keep ? x_ + add * LOG2E : -INFINITY;
                                    }
                                }
                            } else {
                                x_ = -INFINITY;
                            }
                            x[mt][i] = x_;
                            tmax = fmaxf(tmax, x_);
                        }
                    if (__any(tmax > m_run[qt] + RAISE)) raise(qt, tmax);
                    const float mu = (m_run[qt] == -INFINITY) ? 0.f : m_run[qt];
                    float p[2][4];
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) p[mt][i] = exp2_fast(x[mt][i] - mu);  // exp2(-inf) = 0 for excluded keys
                    pb[qt].v = u4{rn_h2(p[0][0], p[0][1]), rn_h2(p[0][2], p[0][3]), rn_h2(p[1][0], p[1][1]), rn_h2(p[1][2], p[1][3])};
                }
                lacc[LM ? qt : 0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones.h, pb[qt].h, lacc[LM ? qt : 0], 0, 0, 0);
                continue;
            }
            float x[2][4];
            float tmax = -INFINITY;
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float x_ = sacc[qt][mt][i] * sl2;
                    if (MM == 2 || !tile_full) {  // workgroup-uniform
                        const int row = trow[mt][i];
                        if (row >= 0 && q_ok[qt]) {
                            if constexpr (MM == 1) {
                                if (!sym_mask_keep(sym, q_l[qt], row)) x_ = -INFINITY;
                            } else if constexpr (MM == 2) {
                                if (vec_ok[mt]) {
                                    if (((mword[mt] >> (8 * i)) & 0xffu) == 0u) x_ = -INFINITY;
                                } else {
                                    float add;
                                    const bool keep = mask_keep(a.mask, b, q_h[qt], q_l[qt], row, a.L, a.T, add);
                                    x_ = keep ? x_ + add * LOG2E : -INFINITY;
                                }
                            }
                        } else {
                            x_ = -INFINITY;
                        }
                    }
                    x[mt][i] = x_;
                    tmax = fmaxf(tmax, x_);
                }
            if (__any(tmax > m_run[qt] + RAISE)) {  // a handful of times per query
                tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
                tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
                const float mn = fmaxf(m_run[qt], tmax);
                const float alpha = (mn == -INFINITY) ? 1.f : exp2_fast(m_run[qt] - mn);
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
                    p[mt][i] = exp2_fast(x[mt][i] - mu);  // exp2(-inf) = 0 for excluded keys
                    psum += p[mt][i];
                }
            l_run[qt] += psum;
            pb[qt].v = pack_p<DT == 1 && VDMA>(p);
        
        }

        // ---- out^T += V^T . P^T: A = V^T rows (tokens 4jj..4jj+3 and 16+4jj..) from LDS -------
#pragma unroll
        for (int d0 = 0; d0 < NDT; d0 += 4) {
            Op8 va[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                if constexpr (VDMA) {  // tokens 8 jj .. 8 jj + 7 of column 16 (d0 + x) + n: one chunk
                    va[x].v = *reinterpret_cast<const u4 *>(&Vs(cur)[(jj * D + 16 * (d0 + x) + n) * 8]);
                } else {
                    const _Float16 *vrow = &Vs(cur)[(16 * (d0 + x) + n) * VS];
                    const u2 lo = *reinterpret_cast<const u2 *>(vrow + 4 * jj);
                    const u2 hi = *reinterpret_cast<const u2 *>(vrow + 16 + 4 * jj);
                    va[x].v = u4{lo.x, lo.y, hi.x, hi.y};
                }
            }
#pragma unroll
            for (int x = 0; x < 4; ++x)
#pragma unroll
                for (int qt = 0; qt < QT; ++qt)
                    oacc[qt][d0 + x] = mfma_qk<(DT == 1 && VDMA) ? 1 : 0>(va[x], pb[qt], oacc[qt][d0 + x]);
        }
        // What was requested at the top of this step has to land before the barrier: it has had the
        // whole step for it, so the wait is short, and an LDS read of the next step never meets a load
        // in flight into its own buffer.  (Leaving the newest LDS request in flight across the
        // barrier, with a third buffer, measured the same.)
        // A plain barrier instead of __syncthreads(): nothing but LDS traffic (drained here) has to
        // be ordered across it.
        wait_older(std::integral_constant<int, 0>{});
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };
    if (tile_lo < tile_hi) {
        dma(tile_lo, 0);
        if constexpr (!VDMA) {
            fetch(tile_lo, setA);
            stage(0, setA);
            if (tile_lo + 1 < tile_hi) fetch(tile_lo + 1, setA);
        }
    }
    wait_older(std::integral_constant<int, 0>{});
    // (the same wait once more in a form the compiler's bookkeeping sees: it then knows that the
    // query operands have arrived, and does not wait for them -- and with them for every load just
    // issued -- inside the loop)
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), others untouched
    __syncthreads();
    // (unrolled by the two buffers, so that every LDS address is a constant plus the lane's)
    for (int tile = tile_lo; tile < tile_hi; tile += 2) {
        step(tile, 0, setA);
        if (tile + 1 >= tile_hi) break;
        step(tile + 1, 1, setA);
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
            float *part = a.workspace + (((size_t)bh * nsplit + split) * R + i) * (D + 2);
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f4 *>(part + 16 * dt + 4 * jj) = oacc[qt][dt];
            if (jj == 0) {
                part[D] = m_run[qt] * 0.6931471805599453f;  // back from the log2 domain
                part[D + 1] = l;
            }
            continue;
        }
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        const size_t ooff = ((size_t)(b * a.Hq + q_h[qt]) * a.L + q_l[qt]) * D;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            const float o0 = oacc[qt][dt][0] * inv, o1 = oacc[qt][dt][1] * inv;
            const float o2 = oacc[qt][dt][2] * inv, o3 = oacc[qt][dt][3] * inv;
            uint2 w;
            if (DT == 0) {
                w.x = rn_h2(o0, o1);
                w.y = rn_h2(o2, o3);
            } else {
                w.x = (uint32_t)Elem<1>::bits(o0) | ((uint32_t)Elem<1>::bits(o1) << 16);
                w.y = (uint32_t)Elem<1>::bits(o2) | ((uint32_t)Elem<1>::bits(o3) << 16);
            }
            *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(a.out) + ooff + 16 * dt + 4 * jj) = w;
        }
    }
}

}  // namespace

hipError_t launch_attend_prefill_fp(const AttendArgs &a, int nsplit, bool wide, hipStream_t s) {
    const Store &st = a.st;
    const int R = (a.Hq / a.Hkv) * a.L;
    const int bm = wide ? 128 : 64;
    dim3 grid((unsigned)((R + bm - 1) / bm) * st.BH * nsplit), block(256);  // linear: the kernel maps ids to tiles
    const bool ident = a.runs.n == 1 && a.runs.row0[0] == 0 && a.runs.phys0[0] == 0;
    const int mm = a.mask.mode == KVHIP_MASK_NONE ? 0 : (a.mask.mode == KVHIP_MASK_ARRAY ? 2 : 1);
#define PF_M(D, DT, QT, MM)                                                                                   \
    do {                                                                                                      \
        if (ident) hipLaunchKernelGGL((prefill_fp_kernel<D, DT, true, QT, MM>), grid, block, 0, s, a, nsplit);  \
        else hipLaunchKernelGGL((prefill_fp_kernel<D, DT, false, QT, MM>), grid, block, 0, s, a, nsplit);       \
    } while (0)
#define PF(D, DT, QT)                        \
    do {                                     \
        if (mm == 0) PF_M(D, DT, QT, 0);     \
        else if (mm == 1) PF_M(D, DT, QT, 1); \
        else PF_M(D, DT, QT, 2);             \
    } while (0)
#define PF_QT(D, DT)                 \
    do {                             \
        if (wide) PF(D, DT, 2);      \
        else PF(D, DT, 1);           \
    } while (0)
#define PF_DT(D)                                  \
    do {                                          \
        if (st.dtype == KVHIP_F16) PF_QT(D, 0);   \
        else PF_QT(D, 1);                         \
    } while (0)
    if (st.Dk == 64) PF_DT(64);
    else if (st.Dk == 80) PF_DT(80);
    else if (st.Dk == 96) PF_DT(96);
    else if (st.Dk == 128) PF_DT(128);
    else if (st.dtype == KVHIP_F16) PF(256, 0, 1);
    else PF(256, 1, 1);
#undef PF_DT
#undef PF_QT
#undef PF
#undef PF_M
    return hipGetLastError();
}

}  // namespace kvhip
