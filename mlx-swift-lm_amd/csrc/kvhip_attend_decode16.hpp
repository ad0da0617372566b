// Split-sequence attention for quantized caches with 9..16 query rows per kv head (the
// speculative-verify shape: 4 new tokens at a GQA ratio of 4) on v_mfma_f32_16x16x32_f16.
//
// With 16 rows the 16x16x32 instruction is filled exactly, at a quarter of the matrix-core
// time the 4-row broadcast contraction of kvhip_attend_decode.hip needs for the same rows.
// Same decomposition otherwise: a workgroup (4 wavefronts) owns a span of 64-token tiles of one
// (batch, kv-head) pair, a wavefront takes every 4th tile, the partials (max, sum, out[D]) of
// the spans are merged by the combine kernel.
//
//   S^T = K . Q^T    A: lane (n, jj) holds 8 codes of the K row of token tok(tb, n), block tb of
//                    four; B: lane (n, jj) holds the same 8 head-dim positions of query row n.
//                    C: lane (n, jj) receives the scores of row n for tokens tok(tb, 4 jj + i).
//   out^T += V^T P^T A: lane (n, jj) holds 8 tokens of head-dim row 16 db + n of the transposed
//                    V tile; B: the probabilities of row n for the same 8 tokens, which are
//                    exactly what the C registers of two score blocks hold: P never moves.
//
// The freedom in both contractions is the order of the contracted index, which only has to agree
// between A and B.  It is chosen so that every operand is a run of whole packed words:
//   * head dim: a quantization group of GS codes is cut in four lane segments (jj) of GS/4
//     codes; step h of the group takes codes 8 h .. 8 h + 7 of each segment, so one instruction
//     stays inside one group and the group's scale can be applied to its accumulator;
//   * tokens: tok(tb, m) = 16 (m / 4) + 4 tb + m % 4, so lane group jj scores tokens
//     16 jj .. 16 jj + 15 and the 8 probabilities it feeds to step u of PV belong to tokens
//     16 jj + 8 u .. + 7 -- one (4-bit) or two (8-bit) whole words of a V tile row.
// Codes become operands as in the 4-row kernel: a masked word is a pair of fp16 subnormals
// code * 2^-24 (high nibbles * 2^-20, compensated by 1/16 on the other operand).
//
// 2-, 3-, 5- and 6-bit codes (rows and V tile rows are plain bit streams, code j at bit j * bits): a lane's
// segment of a group, or its 16 tokens of a V tile row, starts at a bit offset that is a lane constant.  The lane
// loads the whole dwords that cover it, shifts them down once, and cuts each step's 8 codes out at compile-time
// positions, two codes to a register as the same subnormals; element order is the natural one.
#pragma once

#include <type_traits>

#include "kvhip_mask.hpp"

namespace kvhip {

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
union Op8 {
    h8 h;
    u4 v;
};

constexpr int WAVES = 4;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float TWO24 = 16777216.0f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ uint32_t pack_h2(float lo, float hi) { return pk_h2(lo, hi); }
// scale / bias of a raw (scale, bias) pair; for fp16 the widening folds into the consuming fma
template <int DT> __device__ __forceinline__ float sb_scale(uint32_t raw) {
    if (DT == 0) return (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
    return __uint_as_float(raw << 16);
}
template <int DT> __device__ __forceinline__ float sb_bias(uint32_t raw) {
    if (DT == 0) return (float)__builtin_bit_cast(_Float16, (uint16_t)(raw >> 16));
    return __uint_as_float(raw & 0xffff0000u);
}

// 4 bytes per lane from global memory straight into LDS: lane i's land at `lds_wave_base` + 4 i (the base is
// the same for the whole wavefront; address = wave-uniform `base` in scalar registers + the lane's unsigned
// 32-bit byte offset).  Written as assembly: the compiler does not count it among the vector-memory
// operations in flight, which only makes its own waits stricter (such operations complete in order); the
// kernel waits for it by hand (s_waitcnt vmcnt(0)) before it reads what the load fills.
__device__ __forceinline__ void load_dword_to_lds(gptr base, uint32_t lane_off, const void *lds_wave_base) {
    // (the low half of a flat address inside the LDS aperture is the LDS address itself)
    const uint32_t lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds_wave_base);
    const uint64_t b = (uint64_t)base;
    // (readfirstlane returns a signed int: without the casts the low half would be sign-extended over the high one)
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint64_t sb = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(lane_off), "s"(sb), "s"(lds) : "memory", "m0");
}

// 8 codes -> one 8-element operand.  4 bit: one word, element order (c0,c4,c1,c5,c2,c6,c3,c7),
// registers 1 and 3 hold high nibbles (x16).  8 bit: two words, order (c0,c2,c1,c3,c4,c6,c5,c7).
template <int BITS> struct Codes;
template <> struct Codes<4> {
    static constexpr int WORDS = 1;
    static __device__ __forceinline__ Op8 unpack(const uint32_t *w) {
        Op8 o;
        const uint32_t w8 = w[0] >> 8;
        o.v = u4{w[0] & 0x000f000fu, w[0] & 0x00f000f0u, w8 & 0x000f000fu, w8 & 0x00f000f0u};
        return o;
    }
};
template <> struct Codes<8> {
    static constexpr int WORDS = 2;
    static __device__ __forceinline__ Op8 unpack(const uint32_t *w) {
        Op8 o;
        o.v = u4{w[0] & 0x00ff00ffu, (w[0] >> 8) & 0x00ff00ffu, w[1] & 0x00ff00ffu, (w[1] >> 8) & 0x00ff00ffu};
        return o;
    }
};
// operand position p (0..7) -> which of the 8 codes it holds, and whether it is a high nibble
template <int BITS> __device__ __forceinline__ constexpr int code_of(int p) {
    if (BITS == 4) return 2 * (p >> 2) + ((p >> 1) & 1) + 4 * (p & 1);  // (0,4,1,5,2,6,3,7)
    if (BITS == 8) return 4 * (p >> 2) + ((p >> 1) & 1) + 2 * (p & 1);  // (0,2,1,3,4,6,5,7)
    return p;                                                            // bit streams: natural order
}
// A lane's piece of a bit stream: SEGB bits at bit SEGB * jj of a run of GW dwords (a K group, a V tile row).
// The lane loads NWL whole dwords from dword w0(jj) on -- never past the run's end -- and shifts them down by
// sh(jj) bits, which leaves its piece at bit 0 of SEGW dwords.
template <int SEGB, int GW> struct Seg {
    static constexpr int need(int jj) { return (((SEGB * jj) & 31) + SEGB + 31) / 32; }
    static constexpr int imax(int x, int y) { return x > y ? x : y; }
    static constexpr int NWL = imax(imax(need(0), need(1)), imax(need(2), need(3)));
    static constexpr int SEGW = (SEGB + 31) / 32;
    static constexpr int w0(int jj) { return ((SEGB * jj) >> 5) > GW - NWL ? GW - NWL : ((SEGB * jj) >> 5); }
    static constexpr int sh(int jj) { return SEGB * jj - 32 * w0(jj); }
    static constexpr bool ALIGNED = sh(0) == 0 && sh(1) == 0 && sh(2) == 0 && sh(3) == 0;
    static constexpr bool WIDE = sh(0) >= 32 || sh(1) >= 32 || sh(2) >= 32 || sh(3) >= 32;  // (3 bits, group 32)
    static_assert(NWL <= GW && sh(3) < 64 && (!WIDE || NWL == 2), "segment loads stay inside the run");
    static __device__ __forceinline__ int lane_w0(int jj) { return min((SEGB * jj) >> 5, GW - NWL); }
    static __device__ __forceinline__ void normalize(const uint32_t *w, int s, uint32_t (&n)[SEGW]) {
#pragma unroll
        for (int i = 0; i < SEGW; ++i) {
            if constexpr (ALIGNED) n[i] = w[i];
            else if (i + 1 < NWL) n[i] = WIDE ? (uint32_t)((((uint64_t)w[i + 1] << 32) | w[i]) >> s) : __builtin_amdgcn_alignbit(w[i + 1], w[i], (uint32_t)s);
            else n[i] = w[i] >> s;
        }
    }
};
// codes 8 h .. 8 h + 7 of a normalized piece as an operand
template <int BITS, int SEGW> __device__ __forceinline__ Op8 stream_operand(const uint32_t (&n)[SEGW], int h) {
    Op8 o;
    o.v = stream_chunk<BITS, SEGW>(n, h, 0u);
    return o;
}
template <int BITS> __device__ __forceinline__ constexpr bool hi_of(int p) { return BITS == 4 && ((p >> 1) & 1); }

// MM: 0 no mask, 1 index-only mask (causal / window with per-batch bounds), 2 array mask.
// (8-bit codes at D = 256 take more than 256 registers: one workgroup per CU)
// DK / DV: head sizes of keys / queries and of values / outputs (192 and 128 for the multi-head latent attention
// models, equal otherwise).
template <int BITS, int DK, int DV, int GS, int DT, int MM>
__global__ void __launch_bounds__(WAVES * 64, (DK >= 256 && BITS == 8) ? 1 : 2)
decode16_kernel(AttendArgs a, int tiles_total, int tiles_per_wg, int nsplit) {
    constexpr bool GEN = BITS != 4 && BITS != 8;  // bit streams
    using SK = Seg<(GS / 4) * BITS, GS * BITS / 32>;  // a lane's segment of a K group
    using SV = Seg<16 * BITS, 2 * BITS>;              // a lane's 16 tokens of a V tile row
    constexpr int CW = BITS == 8 ? 2 : 1;        // (4 / 8 bits) words per contraction step
    constexpr int GK = DK / GS, GV = DV / GS;    // quantization groups per K row and per V row
    constexpr int SPG = GS / 32;                 // contraction steps per group
    constexpr int KWL = GEN ? SK::NWL : GS * BITS / 8 / 16;  // words per lane, group and K row (segment of GS/4 codes)
    constexpr int NDB = DV / 16;                 // 16-row blocks of out^T
    constexpr int VWL = GEN ? SV::NWL : 16 * BITS / 32;      // words per lane and V row: its 16 tokens
    constexpr int VROW = 64 * BITS / 8;          // bytes of one V tile row
    constexpr int RR = 16;
    // Three or four groups per row (group size 32 at D = 96 / 128, 64 at D = 256), and D = 256 with two: the (scale, bias) pairs of a tile -- 64 tokens
    // x G pairs per side, 2 G registers per token of the lane group if held in registers -- go from global memory
    // straight into LDS one tile ahead and are read from there four tokens at a time when they are used.
    constexpr bool SB_LDS = GK >= 3 || GV >= 3 || DK >= 256;  // (D = 256: the accumulators alone take 64 registers)
    // words between the 64-word pieces the pairs arrive in (G = 2, 4: no lane group's pairs straddle two pieces;
    // the gap keeps the four lane groups' reads on different banks)
    constexpr int SB_PAD_K = (GK == 4 || GK == 2) ? 4 : 0, SB_PAD_V = (GV == 4 || GV == 2) ? 4 : 0;
    constexpr int SB_WORDS_K = GK * (64 + SB_PAD_K), SB_WORDS_V = GV * (64 + SB_PAD_V);
    constexpr int SB_WORDS = SB_LDS ? (SB_WORDS_K > SB_WORDS_V ? SB_WORDS_K : SB_WORDS_V) : 4;
    const Store &st = a.st;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15, jj = lane >> 4;
    int bh = blockIdx.y, split = blockIdx.x;
    int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int r = a.Hq / a.Hkv;
    const int R = r * a.L;
    size_t part_slot = (size_t)bh * nsplit + split;  // where this workgroup's partial goes

    __shared__ float cbuf[WAVES][RR][DV + 2];
    __shared__ __attribute__((aligned(16))) uint32_t sbuf[WAVES][2][2][SB_WORDS];  // [wavefront][tile parity][K, V][pairs]

    // ---- span of this workgroup (as in the 4-row kernel) -----------------------------------
    if constexpr (MM == 1) {
        // a ragged batch whose rows divide their own ranges over the same number of spans: long and short
        // rows are paired on the CUs (balanced_row)
        if (tiles_per_wg == 0 && a.B <= 64 && a.B > 2) {
            b = __builtin_amdgcn_readfirstlane(balanced_row(a.mask, a.B, a.L, a.T, tiles_total, b));
            bh = b * a.Hkv + hk;
            part_slot = (size_t)bh * nsplit + split;
        }
    }
    const SymMask sym = sym_mask_init(a.mask, b, a.L, a.T);
    int tile_begin = split * tiles_per_wg;
    int tile_end = min(tiles_total, tile_begin + tiles_per_wg);
    if constexpr (MM == 1) {
        int vis_lo, vis_hi;
        sym_mask_row_range(sym, vis_lo, vis_hi);
        int t_lo = max(0, vis_lo) >> 6, t_hi = min(tiles_total, (min(vis_hi, a.T - 1) >> 6) + 1);
        if (sym_mask_some_row_empty(sym)) {  // a fully masked row averages over every key
            t_lo = 0;
            t_hi = tiles_total;
        }
        const int per = tiles_per_wg > 0 ? tiles_per_wg
                                         : (max(t_hi - t_lo, 1) + nsplit * WAVES - 1) / (nsplit * WAVES) * WAVES;
        tile_begin = t_lo + split * per;
        tile_end = min(t_hi, tile_begin + per);
    }
    // (wave-uniform by construction; saying so keeps the page walk in scalar registers and scalar loads)
    const int tile0 = __builtin_amdgcn_readfirstlane(tile_begin + wave);
    const int my_tiles = __builtin_amdgcn_readfirstlane(tile0 < tile_end ? (tile_end - tile0 + WAVES - 1) / WAVES : 0);
    int full_lo = 0, full_hi = a.T - 1;  // rows every query row keeps
    if constexpr (MM == 1) {
        sym_mask_full_range(sym, full_lo, full_hi);
        full_hi = min(full_hi, a.T - 1);
    }
    const int row_l = n % a.L, row_rep = n / a.L;  // this lane's query row n = (head rep, position l)
    const bool row_ok = n < R;

    // ---- the step's new row, when it is still to be written (unmasked single-token step) --------
    // Its slot lies in the last tile, which exactly one wavefront of one workgroup reads: that wavefront
    // quantizes the row into the cache before it requests any tile, with the arithmetic of the append kernel,
    // so its own later loads of the tile (and of the tile's scale / bias pairs) see it.  A lane owns the V
    // columns it quantizes; their codes go into the columns' tile rows read-modify-write (a code of a bit
    // stream may lie across two dwords).
    if constexpr (MM == 0) {
        if (a.new_k != nullptr) {  // wave-uniform
            const int slot = a.new_slot, tl = slot >> 6;
            if (tl >= tile_begin && tl < tile_end && ((tl - tile_begin) % WAVES) == wave) {
                const char *krow = static_cast<const char *>(a.new_k) + (size_t)bh * DK * 2;
                const char *vrow = static_cast<const char *>(a.new_v) + (size_t)bh * DV * 2;
                quantize_row_wave_from<DT, BITS>([&](int d) { return Elem<DT>::load(krow, d); }, DK, GS, lane,
                                                 reinterpret_cast<uint32_t *>(const_cast<char *>(k_row_ptr(st, bh, slot))),
                                                 [](int, uint32_t) {}, const_cast<char *>(ksb_row_ptr(st, bh, slot)), nullptr, nullptr);
                char *vcell = const_cast<char *>(v_cell_ptr(st, bh, slot));
                const int bp = v_bitpos<BITS>(slot & (TILE - 1)), sh = bp & 31;
                constexpr uint32_t M = (1u << BITS) - 1u;
                quantize_row_wave_from<DT, BITS>(
                    [&](int d) { return Elem<DT>::load(vrow, d); }, DV, GS, lane, nullptr,
                    [&](int d, uint32_t code) {
                        uint32_t *p = reinterpret_cast<uint32_t *>(vcell + v_row_off(st, slot, d)) + (bp >> 5);
                        p[0] = (p[0] & ~(M << sh)) | (code << sh);
                        if ((32 % BITS) != 0 && sh + BITS > 32) p[1] = (p[1] & ~(M >> (32 - sh))) | (code >> (32 - sh));
                    },
                    const_cast<char *>(vsb_row_ptr(st, bh, slot)), nullptr, nullptr);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            }
        }
    }

    // ---- per-lane addresses inside a tile; tiles of one wavefront are a page apart -----------
    // K block tb, lane (n, jj): row of token tok(tb, n) = 16 (n / 4) + 4 tb + n % 4, segment jj
    // each page is found through the page table (a scalar load per plane pair); the offsets below are
    // the same in every page
    const int tip = tile0 & 3;
    int page_k = my_tiles > 0 ? tile0 >> 2 : 0, page_v = page_k;
    const size_t k_off = (size_t)bh * st.k_cell + (size_t)tip * TILE * st.k_row
                         + (size_t)(16 * (n >> 2) + (n & 3)) * st.k_row + (GEN ? SK::lane_w0(jj) * 4 : jj * (KWL * 4));
    const size_t v_off = (size_t)bh * st.v_cell + (size_t)tip * DV * VROW + (size_t)n * VROW + (GEN ? SV::lane_w0(jj) * 4 : jj * (VWL * 4));
    // (bit streams) how far the lane's piece lies above bit 0 of the dwords it loads
    const int k_sh = (GS / 4) * BITS * jj - 32 * SK::lane_w0(jj), v_sh = 16 * BITS * jj - 32 * SV::lane_w0(jj);
    // (scale, bias) pairs of this lane group's 16 tokens, 16 jj .. 16 jj + 15
    const size_t ksb_off = (size_t)bh * st.ksb_cell + (size_t)(tip * TILE + 16 * jj) * st.ksb_row;
    const size_t vsb_off = (size_t)bh * st.vsb_cell + (size_t)(tip * TILE + 16 * jj) * st.vsb_row;
    // The plane bases of the wavefront's next tile stay wave-uniform (scalar registers) until the loads
    // that use them are formed: the entry of the following page is asked for right after a tile's loads
    // are issued and its latency passes behind the tile's arithmetic.  (Adding the lane's offset as soon
    // as the entry arrived put a wait for the scalar load into every tile: 44 -> 50 us on a ragged
    // batch of 16 rows.)
    gptr kb = as_global(st.pt[page_k].k), vb = as_global(st.pt[page_k].v), ksb_b = as_global(st.pt[page_k].ksb), vsb_b = as_global(st.pt[page_k].vsb);
    int base_next = tile0 * TILE;

    struct Tile {
        uint32_t k[4][GK][KWL];
        uint32_t v[NDB][VWL];
        uint32_t ksb[SB_LDS ? 1 : 16][GK], vsb[SB_LDS ? 1 : 16][GV];  // raw (scale, bias) pairs per token of the lane group
        int base;                          // first slot of the tile
    };
    // (SB_LDS) the pairs of the wavefront's tile number `i`, both sides, into the buffer of that parity; the plane
    // bases walk the page table on their own, one page ahead, like the code planes'
    int page_sb = page_k, sb_issued = 0;
    gptr ksb_n = ksb_b, vsb_n = vsb_b;
    auto dma_sb = [&]() __attribute__((always_inline)) {
        const size_t tile_off = (size_t)tip * TILE;
        const gptr ks = ksb_n + (size_t)bh * st.ksb_cell + tile_off * st.ksb_row;
        const gptr vs = vsb_n + (size_t)bh * st.vsb_cell + tile_off * st.vsb_row;
        const int par = sb_issued & 1;
#pragma unroll
        for (int c = 0; c < GK; ++c) load_dword_to_lds(ks, (uint32_t)(c * 256 + lane * 4), &sbuf[wave][par][0][c * (64 + SB_PAD_K)]);
#pragma unroll
        for (int c = 0; c < GV; ++c) load_dword_to_lds(vs, (uint32_t)(c * 256 + lane * 4), &sbuf[wave][par][1][c * (64 + SB_PAD_V)]);
        ++sb_issued;
        if (sb_issued < my_tiles) {
            ++page_sb;
            ksb_n = as_global(st.pt[page_sb].ksb);
            vsb_n = as_global(st.pt[page_sb].vsb);
        }
    };
    // (SB_LDS) the pairs of tokens 4 tb .. 4 tb + 3 of the lane group, side 0 K (G = GK) / 1 V (G = GV): out[i * G + g]
    auto sb_quad = [&](int par, auto SIDE_, int tb, auto &out) __attribute__((always_inline)) {
        constexpr int side = decltype(SIDE_)::value;
        constexpr int G = side == 0 ? GK : GV, PAD = side == 0 ? SB_PAD_K : SB_PAD_V;
        const int first = 16 * G * jj;  // the lane group's first word among the tile's 64 G
        const u4 *p = reinterpret_cast<const u4 *>(&sbuf[wave][par][side][first + PAD * (first >> 6) + 4 * G * tb]);
#pragma unroll
        for (int e = 0; e < G; ++e) {
            const u4 w = p[e];
            out[4 * e] = w.x; out[4 * e + 1] = w.y; out[4 * e + 2] = w.z; out[4 * e + 3] = w.w;
        }
    };

    int k_loaded = 0, v_loaded = 0;
    auto load_k = [&](Tile &t) __attribute__((always_inline)) {
        const gptr kp = kb + k_off, ksp = ksb_b + ksb_off;
#pragma unroll
        for (int tb = 0; tb < 4; ++tb)
#pragma unroll
            for (int g = 0; g < GK; ++g) {
                const gptr p = kp + (size_t)(4 * tb) * st.k_row + g * (GS * BITS / 8);
                if constexpr (GEN) {  // whole dwords, at dword alignment
#pragma unroll
                    for (int e = 0; e < KWL; ++e) t.k[tb][g][e] = ld_global<uint32_t>(p, e);
                } else if constexpr (KWL == 1) {
                    t.k[tb][g][0] = ld_global<uint32_t>(p);
                } else if constexpr (KWL == 2) {
                    const u2 w = ld_global<u2>(p);
                    t.k[tb][g][0] = w.x; t.k[tb][g][1] = w.y;
                } else {
#pragma unroll
                    for (int e = 0; e < KWL / 4; ++e) {
                        const u4 w = ld_global<u4>(p, e);
                        t.k[tb][g][4 * e] = w.x; t.k[tb][g][4 * e + 1] = w.y;
                        t.k[tb][g][4 * e + 2] = w.z; t.k[tb][g][4 * e + 3] = w.w;
                    }
                }
            }
        // 16 tokens x G pairs of 4 bytes: contiguous rows of G * 4 bytes
        if constexpr (!SB_LDS) {
#pragma unroll
            for (int e = 0; e < 16 * GK / 4; ++e) {
                const u4 w = ld_global<u4>(ksp, e);
                (&t.ksb[0][0])[4 * e] = w.x; (&t.ksb[0][0])[4 * e + 1] = w.y;
                (&t.ksb[0][0])[4 * e + 2] = w.z; (&t.ksb[0][0])[4 * e + 3] = w.w;
            }
        }
        t.base = base_next;
        ++k_loaded;
        if (k_loaded < my_tiles) {  // wave-uniform: the same tile of the next page
            ++page_k;
            kb = as_global(st.pt[page_k].k);
            if constexpr (!SB_LDS) ksb_b = as_global(st.pt[page_k].ksb);
            base_next += PAGE;
        }
    };
    auto load_v = [&](Tile &t) __attribute__((always_inline)) {
        const gptr vp = vb + v_off, vsp = vsb_b + vsb_off;
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
            const gptr p = vp + (size_t)(16 * db) * VROW;
            if constexpr (GEN) {
#pragma unroll
                for (int e = 0; e < VWL; ++e) t.v[db][e] = ld_global<uint32_t>(p, e);
            } else if constexpr (VWL == 2) {
                const u2 w = ld_global<u2>(p);
                t.v[db][0] = w.x; t.v[db][1] = w.y;
            } else {
                const u4 w = ld_global<u4>(p);
                t.v[db][0] = w.x; t.v[db][1] = w.y; t.v[db][2] = w.z; t.v[db][3] = w.w;
            }
        }
        if constexpr (!SB_LDS) {
#pragma unroll
            for (int e = 0; e < 16 * GV / 4; ++e) {
                const u4 w = ld_global<u4>(vsp, e);
                (&t.vsb[0][0])[4 * e] = w.x; (&t.vsb[0][0])[4 * e + 1] = w.y;
                (&t.vsb[0][0])[4 * e + 2] = w.z; (&t.vsb[0][0])[4 * e + 3] = w.w;
            }
        }
        ++v_loaded;
        if (v_loaded < my_tiles) {
            ++page_v;
            vb = as_global(st.pt[page_v].v);
            if constexpr (!SB_LDS) vsb_b = as_global(st.pt[page_v].vsb);
        }
    };

    // ---- query operands (B of S^T) and the group sums of each query row ------------------------
    Op8 qb[GK][SPG];
    float qsum[GK];
    auto load_queries = [&]() __attribute__((always_inline)) {
        // rows past R read row 0 (in bounds) and are zeroed: no branch around the loads, which
        // are one 16-byte piece per contraction step
        const int rep = row_ok ? row_rep : 0, lq = row_ok ? row_l : 0;
        const uint16_t *qrow = reinterpret_cast<const uint16_t *>(a.q) + ((size_t)(b * a.Hq + hk * r + rep) * a.L + lq) * DK;
        u4 raw[GK][SPG];
#pragma unroll
        for (int g = 0; g < GK; ++g)
#pragma unroll
            for (int h = 0; h < SPG; ++h)
                raw[g][h] = *reinterpret_cast<const u4 *>(qrow + GS * g + (GS / 4) * jj + 8 * h);
#pragma unroll
        for (int g = 0; g < GK; ++g) {
            float part = 0.f;
#pragma unroll
            for (int h = 0; h < SPG; ++h) {
                float qv[8];
#pragma unroll
                for (int p = 0; p < 8; ++p) {
                    const int c = code_of<BITS>(p);  // element c of the 8 this step contracts
                    const uint32_t w = raw[g][h][c >> 1];
                    const uint16_t bits16 = (c & 1) ? (uint16_t)(w >> 16) : (uint16_t)w;
                    const float e = DT == 0 ? (float)__builtin_bit_cast(_Float16, bits16) : __uint_as_float((uint32_t)bits16 << 16);
                    const float v = row_ok ? (float)(_Float16)round_dt<DT>(e * a.scale) : 0.f;
                    part += v;
                    qv[p] = hi_of<BITS>(p) ? v * 0.0625f : v;
                }
                qb[g][h].v = u4{pack_h2(qv[0], qv[1]), pack_h2(qv[2], qv[3]), pack_h2(qv[4], qv[5]), pack_h2(qv[6], qv[7])};
            }
            part += __shfl_xor(part, 16);
            part += __shfl_xor(part, 32);
            qsum[g] = part;
        }
    };

    // ---- running state: lane (n, jj) carries row n; m is equal in the four lanes of a row -------
    // (float16 caches, 4-bit codes: the probabilities that meet high nibbles are formed already divided by 16
    // and summed apart -- `l_hi`, `bacc_hi` -- so that no multiply brings them down; they rejoin at the end)
    constexpr bool SPLIT_HI = DT == 0 && BITS == 4;
    float m_run = -INFINITY, l_part = 0.f, bacc[GV], l_hi = 0.f, bacc_hi[GV];
    f4 oacc[NDB];
#pragma unroll
    for (int g = 0; g < GV; ++g) bacc[g] = bacc_hi[g] = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db) oacc[db] = f4{0.f, 0.f, 0.f, 0.f};
    const float fill = finfo_min_dt(DT);

    Op8 pb[GV][2];  // probabilities of the tile in flight: per group (pre-scaled by V's scale), step u

    auto compute_qk_softmax = [&](const Tile &t, int par) __attribute__((always_inline)) {
        // ---- S^T blocks --------------------------------------------------------------------
        f4 sacc[4][GK];
#pragma unroll
        for (int tb = 0; tb < 4; ++tb)
#pragma unroll
            for (int g = 0; g < GK; ++g) {
                sacc[tb][g] = f4{0.f, 0.f, 0.f, 0.f};
                if constexpr (GEN) {
                    uint32_t nk[SK::SEGW];
                    SK::normalize(t.k[tb][g], k_sh, nk);
#pragma unroll
                    for (int h = 0; h < SPG; ++h) {
                        const Op8 ka = stream_operand<BITS, SK::SEGW>(nk, h);
                        sacc[tb][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka.h, qb[g][h].h, sacc[tb][g], 0, 0, 0);
                    }
                } else {
#pragma unroll
                    for (int h = 0; h < SPG; ++h) {
                        const Op8 ka = Codes<GEN ? 4 : BITS>::unpack(&t.k[tb][g][h * CW]);
                        sacc[tb][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka.h, qb[g][h].h, sacc[tb][g], 0, 0, 0);
                    }
                }
            }
        // ---- scores of row n for this lane group's 16 tokens: local token 4 tb + i ---------------
        // (float16 caches keep the rounded scores as float16: the maximum is taken on them and the exponent's
        // multiply-add reads them directly, so they are never widened one by one)
        using XT = typename std::conditional<DT == 0, _Float16, float>::type;
        XT x[16];
#pragma unroll
        for (int tb = 0; tb < 4; ++tb) {
            uint32_t kq[4 * GK];
            if constexpr (SB_LDS) sb_quad(par, std::integral_constant<int, 0>{}, tb, kq);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int tl = 4 * tb + i;
                // q . (s c + b) per group = s (q . c) + b sum(q); the 2^24 of the masked-code operands is
                // taken out of the sum over the groups (one multiply-add instead of one multiply per group)
                float sc_ = 0.f, sb_ = 0.f;
#pragma unroll
                for (int g = 0; g < GK; ++g) {
                    const uint32_t raw = SB_LDS ? kq[i * GK + g] : t.ksb[SB_LDS ? 0 : tl][g];
                    sc_ = __builtin_fmaf(sb_scale<DT>(raw), sacc[tb][g][i], sc_);
                    sb_ = __builtin_fmaf(sb_bias<DT>(raw), qsum[g], sb_);
                }
                x[tl] = (XT)round_dt<DT>(__builtin_fmaf(sc_, TWO24, sb_));
            }
        }
        if (MM == 2 && a.mask.dtype == KVHIP_BOOL && t.base + (TILE - 1) < a.T) {
            // a boolean array over a whole tile: this lane's 16 tokens are 16 consecutive bytes of its
            // query row
            uint32_t mw[4] = {~0u, ~0u, ~0u, ~0u};
            if (row_ok) mask_bool_words<4>(a.mask, b, hk * r + row_rep, row_l, t.base + 16 * jj, mw);
#pragma unroll
            for (int tl = 0; tl < 16; ++tl)
                if (((mw[tl >> 2] >> (8 * (tl & 3))) & 0xffu) == 0u) x[tl] = (XT)fill;
        } else if (MM == 2 || t.base < full_lo || t.base + (TILE - 1) > full_hi) {  // wave-uniform: edge tile
#pragma unroll
            for (int tl = 0; tl < 16; ++tl) {
                const int row = t.base + 16 * jj + tl;  // slots are presented rows
                float s_ = (float)x[tl];
                if (row < a.T) {
                    if constexpr (MM == 1) {
                        if (!sym_mask_keep(sym, row_l, row)) s_ = fill;
                    } else if constexpr (MM == 2) {
                        if (row_ok) {
                            float add;
                            const bool keep = mask_keep(a.mask, b, hk * r + row_rep, row_l, row, a.L, a.T, add);
                            if (!keep) s_ = fill;
                            else if (a.mask.dtype != KVHIP_BOOL) s_ = round_dt<DT>(s_ + add);
                        }
                    }
                } else {
                    s_ = -INFINITY;
                }
                x[tl] = (XT)s_;
            }
        }
        // this lane's largest score: a tree of packed maxima (float16 scores sit two to a register) or of
        // three-operand maxima -- a chain of compares and selects is sixteen dependent steps
        float tmax;
        if constexpr (DT == 0) {
            typedef _Float16 h2v __attribute__((ext_vector_type(2)));
            h2v m2[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) m2[u] = h2v{x[2 * u], x[2 * u + 1]};
#pragma unroll
            for (int w = 4; w >= 1; w >>= 1)
#pragma unroll
                for (int u = 0; u < w; ++u) m2[u] = __builtin_elementwise_max(m2[u], m2[u + w]);
            tmax = fmaxf((float)m2[0].x, (float)m2[0].y);
        } else {
            float m4[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) m4[u] = fmaxf(fmaxf((float)x[4 * u], (float)x[4 * u + 1]), fmaxf((float)x[4 * u + 2], (float)x[4 * u + 3]));
            tmax = fmaxf(fmaxf(m4[0], m4[1]), fmaxf(m4[2], m4[3]));
        }
        // raise the row maximum only when some lane's own maximum exceeds it (rare after the
        // first tiles); it stays equal in the four lanes of a row
        if (__any(tmax > m_run)) {
            tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
            const float mn = fmaxf(m_run, tmax);
            const float alpha = (mn == -INFINITY) ? 1.f : fast_exp2((m_run - mn) * LOG2E);
            m_run = mn;
            l_part *= alpha;
            l_hi *= alpha;
#pragma unroll
            for (int g = 0; g < GV; ++g) {
                bacc[g] *= alpha;
                bacc_hi[g] *= alpha;
            }
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) oacc[db][i] *= alpha;
        }
        const float mu = (m_run == -INFINITY) ? 0.f : m_run;
        const float nmu = -mu * LOG2E;  // (float16: |mu| <= 65504, the product is finite)
        float pv[GV][16];
#pragma unroll
        for (int tb = 0; tb < 4; ++tb) {
            uint32_t vq[4 * GV];
            if constexpr (SB_LDS) sb_quad(par, std::integral_constant<int, 1>{}, tb, vq);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int tl = 4 * tb + i;
                // positions 2, 3, 6, 7 of a 4-bit operand meet high nibbles (x16)
                const bool hi = hi_of<BITS>(tl & 7);
                float p, ps;
                if constexpr (DT == 0) {
                    // one multiply-add on the float16 score; exp2(-inf) = 0 for dead slots
                    ps = fast_exp2(__builtin_fmaf((float)x[tl], LOG2E, (SPLIT_HI && hi) ? nmu - 4.f : nmu));
                    p = ps;
                } else {
                    // (the difference first: a masked score is finfo(T).min, whose product with log2 e overflows for bfloat16)
                    p = fast_exp2((x[tl] - mu) * LOG2E);
                    ps = hi ? p * 0.0625f : p;
                }
                if (SPLIT_HI && hi) l_hi += p;
                else l_part += p;
#pragma unroll
                for (int g = 0; g < GV; ++g) {
                    const uint32_t raw = SB_LDS ? vq[i * GV + g] : t.vsb[SB_LDS ? 0 : tl][g];
                    if (SPLIT_HI && hi) bacc_hi[g] = __builtin_fmaf(p, sb_bias<DT>(raw), bacc_hi[g]);
                    else bacc[g] = __builtin_fmaf(p, sb_bias<DT>(raw), bacc[g]);
                    // (float16: written as a multiply-add so that the widening of the scale folds into it)
                    if constexpr (DT == 0) pv[g][tl] = __builtin_fmaf(sb_scale<DT>(raw), ps, 0.f);
                    else pv[g][tl] = ps * sb_scale<DT>(raw);
                }
            }
        }
#pragma unroll
        for (int g = 0; g < GV; ++g)
#pragma unroll
            for (int u = 0; u < 2; ++u)
                pb[g][u].v = u4{pack_h2(pv[g][8 * u], pv[g][8 * u + 1]), pack_h2(pv[g][8 * u + 2], pv[g][8 * u + 3]),
                                pack_h2(pv[g][8 * u + 4], pv[g][8 * u + 5]), pack_h2(pv[g][8 * u + 6], pv[g][8 * u + 7])};
    };

    auto compute_pv = [&](const Tile &t) __attribute__((always_inline)) {
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
            const int g = (16 * db) / GS;  // a constant once the loop is unrolled
            if constexpr (GEN) {
                uint32_t nv[SV::SEGW];
                SV::normalize(t.v[db], v_sh, nv);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const Op8 va = stream_operand<BITS, SV::SEGW>(nv, u);
                    oacc[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va.h, pb[g][u].h, oacc[db], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const Op8 va = Codes<GEN ? 4 : BITS>::unpack(&t.v[db][u * CW]);
                    oacc[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va.h, pb[g][u].h, oacc[db], 0, 0, 0);
                }
            }
        }
    };

    // one buffer with the halves skewed: V of a tile is requested before its scores, K of the
    // next tile before its PV
    if (my_tiles > 0) {
        Tile buf;
        if constexpr (SB_LDS) dma_sb();
        load_k(buf);
        load_queries();
        for (int done = 0; done < my_tiles; ++done) {
            if constexpr (SB_LDS) {
                // K codes and pairs of this tile have arrived (everything requested so far); the pairs of the next
                // tile go to the other buffer, whose last readers (the tile before this one) are long done
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                load_v(buf);
                if (sb_issued < my_tiles) dma_sb();
            } else {
                load_v(buf);
            }
            compute_qk_softmax(buf, done & 1);
            load_k(buf);
            compute_pv(buf);
        }
    } else {
#pragma unroll
        for (int g = 0; g < GK; ++g) qsum[g] = 0.f;
    }

    // ---- wavefront partial -> LDS: lane (n, jj) holds out^T[d = 16 db + 4 jj + i][row n] ---------
    if constexpr (SPLIT_HI) {
        l_part = __builtin_fmaf(l_hi, 16.f, l_part);
#pragma unroll
        for (int g = 0; g < GV; ++g) bacc[g] = __builtin_fmaf(bacc_hi[g], 16.f, bacc[g]);
    }
    l_part += __shfl_xor(l_part, 16);
    l_part += __shfl_xor(l_part, 32);
#pragma unroll
    for (int g = 0; g < GV; ++g) {
        bacc[g] += __shfl_xor(bacc[g], 16);
        bacc[g] += __shfl_xor(bacc[g], 32);
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        const int g = (16 * db) / GS;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            cbuf[wave][n][16 * db + 4 * jj + i] = oacc[db][i] * TWO24 + bacc[g];
    }
    if (jj == 0) {
        cbuf[wave][n][DV] = m_run;
        cbuf[wave][n][DV + 1] = l_part;
    }
    __syncthreads();
    // ---- merge the 4 wavefronts; a single span writes the output rows, several leave partials ---
    // the weights of a row's four parts once per row (not once per column: an exponential each)
    __shared__ float wrow[WAVES][RR], mrow[RR];
    if (threadIdx.x < WAVES * RR) {
        const int i = threadIdx.x / WAVES, w = threadIdx.x - i * WAVES;
        float mx = -INFINITY;
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2) mx = fmaxf(mx, cbuf[w2][i][DV]);
        const float mw = cbuf[w][i][DV];
        wrow[w][i] = (mw == -INFINITY) ? 0.f : fast_exp2((mw - mx) * LOG2E);
        if (w == 0) mrow[i] = mx;
    }
    __syncthreads();
    if (nsplit == 1) {
        for (int idx = threadIdx.x; idx < R * DV; idx += WAVES * 64) {
            const int i = idx / DV, c = idx - i * DV;
            float v = 0.f, l = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const float wgt = wrow[w][i];
                v += wgt * cbuf[w][i][c];
                l += wgt * cbuf[w][i][DV + 1];
            }
            const int rep = i / a.L, lq = i - rep * a.L;
            Elem<DT>::store(a.out, ((size_t)(b * a.Hq + hk * r + rep) * a.L + lq) * DV + c, l > 0.f ? v / l : 0.f);
        }
        return;
    }
    float *part = a.workspace + part_slot * RR * (DV + 2);
    for (int idx = threadIdx.x; idx < RR * (DV + 2); idx += WAVES * 64) {
        const int i = idx / (DV + 2), c = idx - i * (DV + 2);
        float v;
        if (c == DV) {
            v = mrow[i];
        } else {
            v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) v += wrow[w][i] * cbuf[w][i][c];
        }
        part[idx] = v;
    }
}

}  // namespace

// Launches the 16-row kernel for the plan the caller made (spans as for the 4-row kernel with
// 4 wavefronts); the caller merges the partials when nsplit > 1.
template <int BITS>
hipError_t launch_decode16_bits(const AttendArgs &a, int tiles_total, int tiles_per_wg, int nsplit, hipStream_t s) {
    const Store &st = a.st;
    dim3 grid(nsplit, st.BH), block(WAVES * 64);
    const int mm = a.mask.mode == KVHIP_MASK_NONE ? 0 : (a.mask.mode == KVHIP_MASK_ARRAY ? 2 : 1);
#define D16_M(DK, DV, GS, DT)                                                                                   \
    do {                                                                                                        \
        if (mm == 0) hipLaunchKernelGGL((decode16_kernel<BITS, DK, DV, GS, DT, 0>), grid, block, 0, s, a, tiles_total, tiles_per_wg, nsplit); \
        else if (mm == 1) hipLaunchKernelGGL((decode16_kernel<BITS, DK, DV, GS, DT, 1>), grid, block, 0, s, a, tiles_total, tiles_per_wg, nsplit); \
        else hipLaunchKernelGGL((decode16_kernel<BITS, DK, DV, GS, DT, 2>), grid, block, 0, s, a, tiles_total, tiles_per_wg, nsplit); \
    } while (0)
#define D16_DT(DK, DV, GS)                             \
    do {                                               \
        if (st.dtype == KVHIP_F16) D16_M(DK, DV, GS, 0); \
        else D16_M(DK, DV, GS, 1);                     \
    } while (0)
    if constexpr (BITS == 4 || BITS == 8) {
        // (head size 96 only divides by group size 32; D = 256 keeps 66 KB of partials in LDS -- one workgroup per
        // CU at group size 64, whose instances also need more than 256 registers)
        if (st.Dk == 64 && st.gs == 32) D16_DT(64, 64, 32);
        else if (st.Dk == 64) D16_DT(64, 64, 64);
        else if (st.Dk == 96) D16_DT(96, 96, 32);
        else if (st.Dk == 192 && st.gs == 32) D16_DT(192, 128, 32);
        else if (st.Dk == 192) D16_DT(192, 128, 64);
        else if (st.Dk == 256 && st.gs == 64) D16_DT(256, 256, 64);
        else if (st.Dk == 256) D16_DT(256, 256, 128);
        else if (st.gs == 32) D16_DT(128, 128, 32);
        else if (st.gs == 64) D16_DT(128, 128, 64);
        else D16_DT(128, 128, 128);
    } else {
        // the other code widths: the shapes decode16_stream_shape() lists
        if (st.Dk == 64 && st.gs == 32) D16_DT(64, 64, 32);
        else if (st.Dk == 64) D16_DT(64, 64, 64);
        else if (st.Dk == 96) D16_DT(96, 96, 32);
        else if (st.Dk == 192) D16_DT(192, 128, 64);
        else if (st.Dk == 256) D16_DT(256, 256, 64);
        else if (st.gs == 32) D16_DT(128, 128, 32);
        else if (st.gs == 64) D16_DT(128, 128, 64);
        else D16_DT(128, 128, 128);
    }
#undef D16_DT
#undef D16_M
    return hipGetLastError();
}

}  // namespace kvhip
