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
// how far ahead of their use the matrix-core operands are read from LDS (registers permitting):
// per query-block count (1: 16 query rows per wavefront, 2: 32)
#ifndef KVHIP_PF_VG1
#define KVHIP_PF_VG1 2
#endif
#ifndef KVHIP_PF_VG2
#define KVHIP_PF_VG2 2
#endif
#ifndef KVHIP_PF_NVB1
#define KVHIP_PF_NVB1 2
#endif
#ifndef KVHIP_PF_NVB2
#define KVHIP_PF_NVB2 2
#endif
#ifndef KVHIP_PF_AHEAD1
#define KVHIP_PF_AHEAD1 2
#endif
#ifndef KVHIP_PF_AHEAD2
#define KVHIP_PF_AHEAD2 1
#endif

#ifndef KV_SB
#define KV_SB __builtin_amdgcn_sched_barrier(0)
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
// INVARIANT for anyone who edits this kernel: (1) an iteration ends with vmcnt(0) and a barrier before
// any wavefront reads the buffer the loads fill, and every wavefront of the workgroup runs the same
// iterations with the same requests (which variant of an iteration it runs may differ); (2)
// vector-memory operations of one wavefront complete in order on this hardware -- the compiler's own
// waits for register loads rely on that when an uncounted LDS load sits between them.
// (address = wave-uniform 64-bit `base` in scalar registers + the lane's unsigned 32-bit byte offset)
__device__ __forceinline__ void load_to_lds(const char *base, uint32_t lane_off, const void *lds_wave_base) {
    // (the low half of a flat address inside the LDS aperture is the LDS address itself)
    const uint32_t lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds_wave_base);
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    // (readfirstlane returns a signed int: without the casts the low half would be sign-extended over the high one)
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint64_t sb = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(sb), "s"(lds) : "memory", "m0");
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
__device__ __forceinline__ uint32_t rn_h2(float lo, float hi) { return pk_h2(lo, hi); }    // round to nearest even
__device__ __forceinline__ uint32_t rn_bf2(float lo, float hi) { return pk_bf2(lo, hi); }
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

// c += a . b and c = a . b on the matrix cores.  DT: 0 fp16 operands, 1 bf16 operands.
template <int DT> __device__ __forceinline__ void mfma_acc(f4 &c, const Op8 &a, const Op8 &b) {
    if constexpr (DT == 0) c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, c, 0, 0, 0);
    else c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
}
template <int DT> __device__ __forceinline__ void mfma_new(f4 &c, const Op8 &a, const Op8 &b) {
    c = f4{0.f, 0.f, 0.f, 0.f};
    mfma_acc<DT>(c, a, b);
}
// D = 256 runs 64 query rows per workgroup only: 128 rows need the accumulator registers of
// a whole SIMD lane (one wavefront per SIMD), which measured slower (0.34 ms against 0.29 ms
// for a 512 x 4607 chunk at B4, 8 query heads).
//
// The loop is software-pipelined over the key tiles: iteration t issues S^T(t+1) = K(t+1) Q^T on
// the matrix cores and, between those instructions, the vector-ALU half of the softmax of tile t
// (scale, exp2, rounding to 16 bits), whose scores iteration t-1 left in registers; then
// out^T += V(t)^T P(t)^T; then the mask, the tile maximum and the (rare) raise of the reference
// maximum for tile t+1.  One wavefront so keeps the matrix cores and the vector ALU busy at the
// same time, which the in-order issue of a tile-at-a-time loop (scores -> softmax -> PV, each
// waiting for the one before) cannot.  K is requested two tiles ahead and V one tile ahead, each
// into the buffer of its tile's parity; one barrier per iteration.
// DK and DV are the head sizes of keys / queries and of values / outputs (192 and 128 for the multi-head
// latent attention models, equal otherwise).
template <int DK, int DV, int DT, bool IDENT, int QT, int MM>
__global__ void __launch_bounds__(256, 2)
prefill_fp_kernel(AttendArgs a, int nsplit) {
    constexpr int BM = 64 * QT;
    constexpr int S = (DK + 31) / 32;  // contraction steps over the head dim (the last one partly zero at D = 80)
    constexpr int NDT = DV / 16;   // 16-row tiles of out^T
    constexpr int NCK = (DK + 63) / 64, NCV = (DV + 63) / 64;  // rounds of 256 16-byte chunks, for K and for V
    constexpr int CHK = 4 * DK, CHV = 4 * DV;  // 16-byte chunks of a tile's K and of its V; multiples of 64
    static_assert(DK % 16 == 0 && DV % 16 == 0, "out^T is built from 16-row tiles");
    // A head size that is not a multiple of 32 (80): the last contraction step reads K chunks past the
    // row -- the unused tail that the repeated loads fill with finite values -- against query
    // operands that are zero there.
    static_assert(4 * S * BN <= NCK * 256, "the padded contraction stays inside the staged buffer");
    // K and V tiles move from global memory straight into LDS (no registers, no LDS store
    // instructions): per parity of the tile one buffer for K, the tile's 16-byte chunks in page order
    // [8-element chunk][token], and one for V, [8-token chunk][column].  bf16 caches keep K and V as
    // bf16: the probabilities are rounded to bf16 for the PV matrix-core instruction (the reference's
    // softmax output is an array of the cache's dtype as well).
    // 16-bit elements reserved for a tile's K (and for its V): whole rounds of 256 chunks.  With a head
    // size that is not a multiple of 64 (80, 96) the last round is partly empty: its wavefronts past the
    // tile's last chunk repeat that chunk into the unused tail, so that every wavefront issues the same
    // number of loads.
    constexpr int KSZ = NCK * 256 * 8, VSZ = NCV * 256 * 8;
    __shared__ __attribute__((aligned(16))) uint16_t KV0[KSZ + VSZ], KV1[KSZ + VSZ];
    auto Ks = [&](int par) __attribute__((always_inline)) -> uint16_t * { return par == 0 ? KV0 : KV1; };
    auto Vs = [&](int par) __attribute__((always_inline)) -> uint16_t * { return (par == 0 ? KV0 : KV1) + KSZ; };
    __shared__ int rows_s[2][BN];
    __shared__ int full_s[2];
    __shared__ int seg_lo_s[MAXRUNS], seg_hi_s[MAXRUNS], nseg_s;  // tile segments to visit (ring presentations)

    const Store &st = a.st;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
            const int xcd = id & 7;
            int j = id >> 3;
            // A grid of exactly two workgroups per CU is resident all at once and gets no balancing from the
            // order of the ids.  Under a causal or window mask the two workgroups of a CU -- 32 apart among the
            // 64 of their XCD -- then take a long and a short query block: the second 32 count backwards.
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
    // Under a causal or window mask the later query blocks see more keys: they are given the lower
    // workgroup ids, which the hardware starts first, so that the launch does not end on its longest blocks.
    if (MM == 1) blk_x = nblk - 1 - blk_x;
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int row0 = blk_x * BM + wave * 16 * QT;  // first query row of this wavefront
    const SymMask sym = sym_mask_init(a.mask, b, a.L, a.T);
    // Scores enter the softmax as exp2(s * ef - m) with ef = |scale| log2 e > 0 -- a negative scale
    // flips the sign of the query operands instead (exact), a zero one becomes a vanishing positive
    // factor -- so that the maximum can be taken on the raw scores and the scale folds into one
    // multiply-add.  Under an array mask the mask step leaves s * ef (+ the additive term) in the
    // score registers and the factor is 1.
    // fp16 caches up to D = 128: the denominators ride on the matrix cores (lacc = ones . P^T sums the
    // same rounded probabilities the numerator uses; all 16 rows of the block hold the same sums).
    // D = 256 has no registers to spare, and bf16 keeps float32 denominators.
    constexpr bool LM = DK <= 128 && DV <= 128 && DT == 0 && KVHIP_PREFILL_LM;
    const bool flip = a.scale < 0.f;
    const float sl2 = fmaxf(fabsf(a.scale) * LOG2E, 1e-30f);
    const float ef = MM == 2 ? 1.f : sl2;

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
            reinterpret_cast<const uint16_t *>(a.q) + ((size_t)(b * a.Hq + q_h[qt]) * a.L + q_l[qt]) * DK + 8 * jj);
#pragma unroll
        for (int s = 0; s < S; ++s) {
            u4 w = (q_ok[qt] && (DK % 32 == 0 || 32 * s + 8 * jj < DK)) ? qp[4 * s] : u4{0, 0, 0, 0};
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
    // The tiles to visit, in slot order, as up to NSEG segments; position v of the visiting order is tile
    // vt_of(v).  With slots in presented order that is the one range found above.  A ring presented
    // through a run table keeps its rows in rotated order, so the rows no query of this block can see
    // (older than the window, newer than the block) lie somewhere inside the slot range: thread 0 maps
    // the visible row range through every run to slot tiles, sorts and merges them (a few dozen scalar
    // steps, once per workgroup), and whole tiles of invisible rows are never requested -- 14 of 144
    // tiles for a 512-row chunk over a 4096-row window.
    constexpr int NSEG = 4;
    int seg_start[NSEG], seg_cnt[NSEG];
#pragma unroll
    for (int k = 0; k < NSEG; ++k) seg_start[k] = seg_cnt[k] = 0;
    seg_start[0] = tile_lo;
    seg_cnt[0] = max(tile_hi - tile_lo, 0);
    if constexpr (!IDENT && MM == 1) {
        if (tid == 0) {
            const int i_first = blk_x * BM, i_last = min(R, i_first + BM) - 1;
            const bool spans = (i_first / a.L) != (i_last / a.L);
            const int l_min = spans ? 0 : i_first % a.L, l_max = spans ? a.L - 1 : i_last % a.L;
            int vis_lo = 0, vis_hi = a.T - a.L + l_max;  // rows some query of the block may see
            if (sym.mode != KVHIP_MASK_CAUSAL) {
                vis_lo = sym.pad_b;
                vis_hi = min(sym.offset + l_max, sym.len_b - 1);
                if (sym.window > 0) vis_lo = max(vis_lo, sym.offset + l_min - sym.window + 1);
            }
            vis_lo = max(vis_lo, 0);
            vis_hi = min(vis_hi, a.T - 1);
            int ns = 0;
#pragma unroll
            for (int i = 0; i < MAXRUNS; ++i) {
                if (i < a.runs.n) {
                    const int r_lo = max(vis_lo, a.runs.row0[i]), r_hi = min(vis_hi, a.runs.row0[i] + a.runs.len[i] - 1);
                    if (r_lo <= r_hi) {
                        const int t_lo = (a.runs.phys0[i] + r_lo - a.runs.row0[i]) / BN;
                        const int t_hi = (a.runs.phys0[i] + r_hi - a.runs.row0[i]) / BN;
                        int pos = ns;  // insertion by first tile
                        while (pos > 0 && seg_lo_s[pos - 1] > t_lo) {
                            seg_lo_s[pos] = seg_lo_s[pos - 1];
                            seg_hi_s[pos] = seg_hi_s[pos - 1];
                            --pos;
                        }
                        seg_lo_s[pos] = t_lo;
                        seg_hi_s[pos] = t_hi;
                        ++ns;
                    }
                }
            }
            int m = 0;  // merge what overlaps or touches
            for (int i = 0; i < ns; ++i) {
                if (m > 0 && seg_lo_s[i] <= seg_hi_s[m - 1] + 1) {
                    seg_hi_s[m - 1] = max(seg_hi_s[m - 1], seg_hi_s[i]);
                } else {
                    seg_lo_s[m] = seg_lo_s[i];
                    seg_hi_s[m] = seg_hi_s[i];
                    ++m;
                }
            }
            if (m > NSEG) {  // more pieces than are kept: one range over all of them (nothing wrong, nothing skipped)
                seg_hi_s[0] = seg_hi_s[m - 1];
                m = 1;
            }
            nseg_s = m;
        }
        __syncthreads();
        const int m = __builtin_amdgcn_readfirstlane(nseg_s);
#pragma unroll
        for (int k = 0; k < NSEG; ++k) {
            const int lo = k < m ? __builtin_amdgcn_readfirstlane(seg_lo_s[k]) : 0;
            const int hi = k < m ? __builtin_amdgcn_readfirstlane(seg_hi_s[k]) : -1;
            seg_start[k] = lo;
            seg_cnt[k] = hi - lo + 1;
        }
    }
    auto vt_of = [&](int v) __attribute__((always_inline)) -> int {
        int t = seg_start[0] + v, rem = v - seg_cnt[0];
#pragma unroll
        for (int k = 1; k < NSEG; ++k) {
            if (rem >= 0) t = seg_start[k] + rem;
            rem -= seg_cnt[k];
        }
        return t;
    };
    int v_lo = 0, v_hi = 0;
#pragma unroll
    for (int k = 0; k < NSEG; ++k) v_hi += seg_cnt[k];
    // optional split of the visiting order (small grids): each part leaves an
    // unnormalised partial per query row, merged by the decode path's combine kernel
    if (nsplit > 1) {
        const int span = (v_hi + nsplit - 1) / nsplit;
        v_lo = split * span;
        v_hi = min(v_hi, v_lo + span);
    }

    // ---- requests -------------------------------------------------------------------------
    // direct global -> LDS: lane i of a wavefront's load lands at the wavefront's LDS base + 16 i, so
    // chunk c = e * 256 + tid goes to slot c of the buffer.  K slot (chunk cc, position pos) takes
    // token 8 ((pos & 15) / 4) + 4 (pos / 16) + pos % 4, the order in which the S^T accumulators of one
    // lane cover the eight tokens of one V chunk (so K operand reads are contiguous across lanes and P
    // never moves), and V slots are the page's own order.
    // A tile of 32 slots inside its page cell (16-bit elements): the 64-token tile t64 starts at
    // t64 * 64 * DK * 2 bytes in the K plane and t64 * 64 * DV * 2 in the V plane; its K chunk (cc, token) lies at
    // (cc * 64 + token) * 16, its V chunk (8-token chunk tc, column) at (tc * DV + column) * 16.
    const size_t cell_k = (size_t)bh * st.k_cell, cell_v = (size_t)bh * st.v_cell;
    PageCursor page_k(st, min(vt_of(v_lo) * BN, max(a.slots - 1, 0))), page_v = page_k;
    // the lane's byte offsets inside a tile, one per round of 256 chunks
    uint32_t koff[NCK], voff[NCV];
#pragma unroll
    for (int e = 0; e < NCK; ++e) {
        const int c = min(e * 256 + tid, CHK - 1);
        const int pos = c % BN;
        const int tok = 8 * ((pos & 15) >> 2) + 4 * (pos >> 4) + (pos & 3);
        koff[e] = (uint32_t)((c / BN) * (TILE * 16) + tok * 16);
    }
#pragma unroll
    for (int e = 0; e < NCV; ++e) voff[e] = (uint32_t)(min(e * 256 + tid, CHV - 1) * 16);
    auto dma_k = [&](int tile, int par) __attribute__((always_inline)) {
        const int slot0 = tile * BN;
        if (wave == (tile & 3) && lane < BN) {  // the wavefronts take this in turn
            const int pos = lane;
            const int slot = slot0 + 8 * ((pos & 15) >> 2) + 4 * (pos >> 4) + (pos & 3);
            int row;
            if (IDENT) row = slot;
            else row = slot < a.slots ? slot_to_row(a.runs, slot) : -1;
            row = (row >= 0 && row < a.T) ? row : -1;
            rows_s[par][pos] = row;  // the row of the token in K slot `pos`
            const bool full = __all(row >= keep_lo && row <= keep_hi);  // (the 32 active lanes)
            if (lane == 0) full_s[par] = full;
        }
        const int t = slot0 & (PAGE - 1);
        const char *kbase = page_k.at(st, slot0).k + cell_k + (size_t)(t >> 6) * (TILE * DK * 2) + (t & 63) * 16;
#pragma unroll
        for (int e = 0; e < NCK; ++e) {
            // whole rounds differ by a constant, which goes to the scalar base; a partly empty last
            // round (its tail repeats the tile's last chunk) keeps its own lane offsets
            if (DK % 64 == 0) load_to_lds(kbase + e * 8 * (TILE * 16), koff[0], &Ks(par)[(e * 256 + 64 * wave) * 8]);
            else load_to_lds(kbase, koff[e], &Ks(par)[(e * 256 + 64 * wave) * 8]);
        }
    };
    auto dma_v = [&](int tile, int par) __attribute__((always_inline)) {
        const int slot0 = tile * BN;
        const int t = slot0 & (PAGE - 1);
        const char *vbase = page_v.at(st, slot0).v + cell_v + (size_t)(t >> 6) * (TILE * DV * 2) + ((t & 63) >> 3) * (DV * 16);
#pragma unroll
        for (int e = 0; e < NCV; ++e) {
            if (DV % 64 == 0) load_to_lds(vbase + e * 256 * 16, voff[0], &Vs(par)[(e * 256 + 64 * wave) * 8]);
            else load_to_lds(vbase, voff[e], &Vs(par)[(e * 256 + 64 * wave) * 8]);
        }
    };
    auto wait_all_loads = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

    // ---- S^T = K . Q^T of one tile: acc[qt][mt] rows = tokens 16 mt + 4 jj + i, column = query n -----
    // operand reads: K slot (chunk 4 s + jj, position 16 mt + n)
    auto read_k = [&](int par, int s, Op8 (&ka)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
            ka[mt].v = *reinterpret_cast<const u4 *>(&Ks(par)[((4 * s + jj) * BN + 16 * mt + n) * 8]);
    };

    // ---- mask of a tile whose scores are in `sc` (raw): excluded keys become -inf; under an array
    // mask the scores are scaled here and additive terms added -----------------------------------
    // An index-only mask (causal, window, per-batch lengths and left padding) keeps, for one query, an
    // interval of key rows: [q_lo, q_lo + q_span] per query block of this lane (empty for a query row
    // past the end), tested with one unsigned comparison per key.
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
            const bool any = q_ok[qt] && hi >= lo;
            q_lo[qt] = any ? lo : 0;
            q_span[qt] = any ? (uint32_t)(hi - lo) : 0u;
            if (!any) q_lo[qt] = 0x40000000;  // no row reaches it: row - q_lo wraps to a huge unsigned value
        }
    }
    auto apply_mask = [&](int par, f4 (&sc)[QT][2]) __attribute__((always_inline)) {
        int trow[2][4];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) trow[mt][i] = rows_s[par][16 * mt + 4 * jj + i];  // by K slot; -1: no row
        if constexpr (MM != 2) {
#pragma unroll
            for (int qt = 0; qt < QT; ++qt)
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        bool keep;
                        if constexpr (MM == 1) keep = (uint32_t)(trow[mt][i] - q_lo[qt]) <= q_span[qt];
                        else keep = trow[mt][i] >= 0 && q_ok[qt];
                        sc[qt][mt][i] = keep ? sc[qt][mt][i] : -INFINITY;
                    }
            return;
        }
        // a boolean array mask is read four keys at a time where this lane's four rows are consecutive
        [[maybe_unused]] bool vec_ok[2] = {false, false};
        if constexpr (MM == 2) {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
                vec_ok[mt] = a.mask.dtype == KVHIP_BOOL && trow[mt][0] >= 0 && trow[mt][3] == trow[mt][0] + 3 &&
                             trow[mt][1] == trow[mt][0] + 1 && trow[mt][2] == trow[mt][0] + 2;
        }
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
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float x_ = sc[qt][mt][i] * sl2;
                    const int row = trow[mt][i];
                    bool keep = row >= 0 && q_ok[qt];
                    if constexpr (MM == 2) {
                        if (keep) {
                            if (vec_ok[mt]) {
                                keep = ((mword[mt] >> (8 * i)) & 0xffu) != 0u;
                            } else {
                                float add;
                                keep = mask_keep(a.mask, b, q_h[qt], q_l[qt], row, a.L, a.T, add);
                                x_ += add * LOG2E;
                            }
                        }
                    }
                    sc[qt][mt][i] = keep ? x_ : -INFINITY;
                }
        }
    };

    // ---- tile maximum and the reference maximum ---------------------------------------------
    // Scores stay in the log2 domain: x = s * ef, p = exp2(x - m).  m is a reference value rather than
    // the exact running maximum: it is the same in the four lanes that share a query and is raised (to
    // the maximum seen) only when a score exceeds it by more than RAISE, so p stays below 2^RAISE
    // (exact in fp16, whose relative precision does not depend on magnitude) and the accumulators are
    // rescaled a handful of times per query, not on every tile that happens to hold a new maximum.
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
    // whether the tile whose scores are in `sc` exceeds some query's reference maximum by more than
    // RAISE (wavefront-uniform; a handful of times per query)
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

    // ---- one iteration: tile `tile` (parity PAR) has its scores in `sc`; `sn` receives tile + 1's ---
    // (MASKED: tile + 1 needs its mask evaluated -- a variant of the whole iteration rather than a
    // branch inside it, so that the scores have one definition per variant and the paths join
    // without register copies)
    // The iteration itself never touches the reference maxima or rescales the accumulators: it only
    // reports (`need`) that tile + 1 calls for it, and the loop below leaves its fast part to do so.
    // With the rescaling inside the fast loop the compiler joined the rescaled and the untouched
    // accumulators through register copies on the path that does not rescale: 36 moves per query block
    // and tile, and spills.
    auto body = [&](auto HAS_NEXT_, auto PAR_, auto MASKED_, int tile, f4 (&sc)[QT][2], f4 (&sn)[QT][2], bool &need) __attribute__((always_inline)) {
        constexpr bool HAS_NEXT = decltype(HAS_NEXT_)::value;
        constexpr int PAR = decltype(PAR_)::value;
        constexpr bool MASKED = decltype(MASKED_)::value;
        // the buffers requested into were last read in the previous iteration, which ended with a barrier
        if (tile + 2 < v_hi) dma_k(vt_of(tile + 2), PAR);  // (`tile`: the position in the visiting order)
        if constexpr (HAS_NEXT) dma_v(vt_of(tile + 1), PAR ^ 1);

        float negmu[QT], pr[QT][2][4];
        Op8 pb[QT];
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) negmu[qt] = (m_run[qt] == -INFINITY) ? 0.f : -m_run[qt];
        // probability `idx` of this lane: query block idx / 8, accumulator idx % 8
        // (the rounding of a pair of probabilities to 16 bits trails their exp2 by two probabilities, so
        // that it does not wait for a result just asked for)
        auto round_pair = [&](int idx) __attribute__((always_inline)) {  // idx: the odd member of the pair
            const int qt = idx >> 3, mt = (idx >> 2) & 1, i = idx & 3;
            const float p0 = pr[qt][mt][i - 1], p1 = pr[qt][mt][i];
            if constexpr (!LM) l_run[qt] += p0 + p1;
            pb[qt].v[2 * mt + (i >> 1)] = DT == 1 ? rn_bf2(p0, p1) : rn_h2(p0, p1);
        };
        constexpr int NP = 8 * QT;      // probabilities per lane and tile
        auto softmax_slice = [&](int idx) __attribute__((always_inline)) {
            const int qt = idx >> 3, mt = (idx >> 2) & 1, i = idx & 3;
            pr[qt][mt][i] = exp2_fast(__builtin_fmaf(sc[qt][mt][i], ef, negmu[qt]));  // exp2(-inf) = 0 for excluded keys
            if ((idx & 1) && idx >= 3) round_pair(idx - 2);
            if (idx == NP - 1) round_pair(idx);
        };
        // V operands (16 columns each) are read in groups of VG, NVB - 1 groups ahead of their use
        constexpr int VG = QT == 1 ? KVHIP_PF_VG1 : KVHIP_PF_VG2;
        constexpr int NVB = QT == 1 ? KVHIP_PF_NVB1 : KVHIP_PF_NVB2;
        constexpr int NG = (NDT + VG - 1) / VG;
        Op8 va[NVB][VG];
        auto read_v = [&](int g, Op8 (&dst)[VG]) __attribute__((always_inline)) {
#pragma unroll
            for (int x = 0; x < VG; ++x)
                if (VG * g + x < NDT)  // tokens 8 jj .. 8 jj + 7 of column 16 (VG g + x) + n: one chunk
                    dst[x].v = *reinterpret_cast<const u4 *>(&Vs(PAR)[(jj * DV + 16 * (VG * g + x) + n) * 8]);
        };
        if constexpr (HAS_NEXT) {
            constexpr int NM = 2 * S * QT;  // matrix-core instructions of the next tile's scores
            // K operands are asked for AHEAD contraction steps ahead, V's first group near the end
            constexpr int AHEAD = QT == 1 ? KVHIP_PF_AHEAD1 : KVHIP_PF_AHEAD2;
            constexpr int KA = S < AHEAD + 1 ? S : AHEAD + 1;
            Op8 ka[KA][2];
#pragma unroll
            for (int s = 0; s < (S < AHEAD ? S : AHEAD); ++s) read_k(PAR ^ 1, s, ka[s % KA]);
            KV_SB;
#pragma unroll
            for (int k = 0; k < NM; ++k) {
                // 2 QT independent accumulator chains, taken in turn
                const int s = k / (2 * QT), mt = (k / QT) & 1, qt = k % QT;
                if (k % (2 * QT) == 0 && s + AHEAD < S) read_k(PAR ^ 1, s + AHEAD, ka[(s + AHEAD) % KA]);
                if (k == (NM > 2 * QT ? NM - 2 * QT : 0)) {
#pragma unroll
                    for (int g = 0; g < NVB - 1 && g < NG; ++g) read_v(g, va[g]);
                }
                if (s == 0) mfma_new<DT>(sn[qt][mt], ka[s % KA][mt], qop[qt][s]);
                else mfma_acc<DT>(sn[qt][mt], ka[s % KA][mt], qop[qt][s]);
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

        // ---- out^T += V^T . P^T: A = V^T chunks from LDS, B = the probabilities where they are ----
        if constexpr (LM) {
#pragma unroll
            for (int qt = 0; qt < QT; ++qt)
                mfma_acc<0>(lacc[LM ? qt : 0], ones, pb[qt]);
        }
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            if (g + NVB - 1 < NG) read_v(g + NVB - 1, va[(g + NVB - 1) % NVB]);
#pragma unroll
            for (int x = 0; x < VG; ++x)
                if (VG * g + x < NDT) {
#pragma unroll
                    for (int qt = 0; qt < QT; ++qt)
                        mfma_acc<DT>(oacc[qt][VG * g + x], va[g % NVB][x], pb[qt]);
                }
        }

        need = false;
        if constexpr (HAS_NEXT) {
            if constexpr (MASKED) apply_mask(PAR ^ 1, sn);
            KV_SB;  // (tile_max_raw: not before the matrix-core instructions above)
            need = needs_raise(sn);
        }
        // What was requested at the top has to land before the barrier: it has had the whole
        // iteration for it, so the wait is short, and no LDS read of the next iteration meets a load
        // in flight into its buffer.  A plain barrier instead of __syncthreads(): nothing but LDS
        // traffic (drained here) has to be ordered across it.
        wait_all_loads();
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };

    if (v_lo < v_hi) {
        dma_k(vt_of(v_lo), 0);
        dma_v(vt_of(v_lo), 0);
        if (v_lo + 1 < v_hi) dma_k(vt_of(v_lo + 1), 1);
    }
    wait_all_loads();
    // (the same wait once more in a form the compiler's bookkeeping sees: it then knows that the
    // query operands have arrived, and does not wait for them -- and with them for every load just
    // issued -- inside the loop)
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), others untouched
    __syncthreads();
    if (v_lo < v_hi) {
        f4 sa[QT][2], sb[QT][2];
        {  // scores of the first tile
#pragma unroll
            for (int s = 0; s < S; ++s) {
                Op8 ka[2];
                read_k(0, s, ka);
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int qt = 0; qt < QT; ++qt) {
                        if (s == 0) mfma_new<DT>(sa[qt][mt], ka[mt], qop[qt][s]);
                        else mfma_acc<DT>(sa[qt][mt], ka[mt], qop[qt][s]);
                    }
            }
            if (MM == 2 || full_s[0] == 0) apply_mask(0, sa);
            do_raise(sa);
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // K buffer 0 is free again
        using T_ = std::true_type;
        using F_ = std::false_type;
        using P0 = std::integral_constant<int, 0>;
        using P1 = std::integral_constant<int, 1>;
        int tile = v_lo;  // position in the visiting order
        // one iteration with the variant chosen at run time; false after the last tile
        auto iterate = [&](auto PAR_, f4 (&sc)[QT][2], f4 (&sn)[QT][2], bool &need) __attribute__((always_inline)) -> bool {
            constexpr int PAR = decltype(PAR_)::value;
            const bool has_next = tile + 1 < v_hi;
            // whether tile + 1 needs its mask evaluated (workgroup-uniform): with slots in presented
            // order a comparison of its ends with the rows every query keeps, else the flag its
            // request left in LDS -- asked for before the requests below are formed, which hide its latency
            bool masked = true;
            if constexpr (MM != 2) {
                if constexpr (IDENT) masked = !(vt_of(tile + 1) * BN >= keep_lo && vt_of(tile + 1) * BN + (BN - 1) <= keep_hi);
                else masked = full_s[PAR ^ 1] == 0;
            }
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
            // the fast loop: two iterations (one per buffer parity) per round, left when a tile's scores
            // call for a higher reference maximum -- after an even number of iterations (`odd` false:
            // the next tile's scores are in sa) or an odd one (in sb)
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
            if (odd) {  // back to an even count through one iteration outside the fast loop
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
                w.x = rn_h2(o0, o1);
                w.y = rn_h2(o2, o3);
            } else {
                w.x = rn_bf2(o0, o1);
                w.y = rn_bf2(o2, o3);
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
#define PF_M(DK, DV, DT, QT, MM)                                                                                   \
    do {                                                                                                      \
        if (ident) hipLaunchKernelGGL((prefill_fp_kernel<DK, DV, DT, true, QT, MM>), grid, block, 0, s, a, nsplit);  \
        else hipLaunchKernelGGL((prefill_fp_kernel<DK, DV, DT, false, QT, MM>), grid, block, 0, s, a, nsplit);       \
    } while (0)
#define PF2(DK, DV, DT, QT)                        \
    do {                                     \
        if (mm == 0) PF_M(DK, DV, DT, QT, 0);     \
        else if (mm == 1) PF_M(DK, DV, DT, QT, 1); \
        else PF_M(DK, DV, DT, QT, 2);             \
    } while (0)
#define PF(D, DT, QT) PF2(D, D, DT, QT)
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
    // keys of 192 with values of 128 (multi-head latent attention): 64 query rows per workgroup
    if (st.Dk == 192 && st.Dv == 128) {
        if (st.dtype == KVHIP_F16) PF2(192, 128, 0, 1);
        else PF2(192, 128, 1, 1);
    } else if (st.Dk == 64) PF_DT(64);
    else if (st.Dk == 80) PF_DT(80);
    else if (st.Dk == 96) PF_DT(96);
    else if (st.Dk == 128) PF_DT(128);
    else if (st.dtype == KVHIP_F16) PF(256, 0, 1);
    else PF(256, 1, 1);
#undef PF_DT
#undef PF_QT
#undef PF
#undef PF2
#undef PF_M
    return hipGetLastError();
}

}  // namespace kvhip
