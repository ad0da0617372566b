// Quantize-on-append of whole 64-token tiles: the element functions, the tile body and its two kernels,
// and the launchers of one code width (instantiated per width in kvhip_io.hip and kvhip_quant_tile_other.hip).
#pragma once
#include "kvhip_device.hpp"

namespace kvhip {

namespace {

// Element d of a row at position `pos` after the rotary embedding, rounded to the row's dtype
// (what the reference hands to the cache: `applyRotaryPosition` runs before `update`,
// Llama.swift:58-62).  The angle is the float32 product of position * scale and the inverse
// frequency exp(-i * log(base) / half), or 1 / freqs[i].
template <int DT>
__device__ __forceinline__ float rope_elem(const RopeDev &r, const void *row, int d, int pos) {
    const float x = Elem<DT>::load(row, d);
    if (d >= r.dims) return x;
    const int half = r.dims >> 1;
    int i, partner;
    bool first;
    if (r.traditional) {
        i = d >> 1;
        partner = d ^ 1;
        first = (d & 1) == 0;
    } else {
        first = d < half;
        i = first ? d : d - half;
        partner = first ? d + half : d - half;
    }
    // the inverse frequency is formed in double and rounded once, so that it does not depend on
    // one exp implementation's last float32 bit (a position of 10^5 turns one such bit into 10^-2 rad)
    const float inv = r.freqs ? 1.0f / r.freqs[i] : (float)exp(-(double)i * r.log_base_over_half);
    const float theta = ((float)pos * r.scale) * inv;
    float sn, cs;
    sincosf(theta, &sn, &cs);
    const float y = Elem<DT>::load(row, partner);
    const float v = first ? x * cs - y * sn : y * sn + x * cs;
    return round_dt<DT>(v);
}
__device__ __forceinline__ int rope_pos(const RopeDev &r, int bh, int l) {
    return (r.batch_pos ? r.batch_pos[bh / r.H] : r.pos0) + l;
}

// ---- whole 64-token tiles (prompt-sized appends) -----------------------------------------
// The per-row kernels above fetch one element per lane and wait for every row in turn; for
// many rows that is bound by load latency.  Here a workgroup takes one whole tile of one
// (batch, kv-head): every thread first requests all of its 16-byte chunks of the 64 new K and
// V rows, then quantizes / copies eight elements at a time.  Values, rounding and the
// rotation are those of the per-row kernels (the same element functions).
typedef uint32_t u4v __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ void unpack8(const u4v &raw, const void *row, int d0, const RopeDev &rope, int pos,
                                        float (&w)[8]) {
    if (rope.dims > 0 && d0 < rope.dims) {
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = rope_elem<DT>(rope, row, d0 + j, pos);
        return;
    }
    const uint32_t u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (DT == 0) {
            w[2 * j] = __half2float(__ushort_as_half((unsigned short)(u[j] & 0xffffu)));
            w[2 * j + 1] = __half2float(__ushort_as_half((unsigned short)(u[j] >> 16)));
        } else {
            w[2 * j] = __uint_as_float(u[j] << 16);
            w[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u);
        }
    }
}

// Codes of the eight elements a thread holds, as integer-valued floats in [0, 2^BITS - 1], from
// the parameters of their group; `inv` is the hardware reciprocal of `scale`.
// code = rint((w - bias) / scale), clamped.  The quotient is first formed with the reciprocal
// (one ulp): product and reciprocal together put it within 2^-22 relative, so within 2^-14
// absolute (|quotient| <= 2^8), of the correctly rounded quotient, which can only change the
// rounded integer when the quotient sits that close to a half-integer.  Those elements (about
// one in 10^4) are redone with the exact division, so the codes are the reference's bit for bit.
// INVARIANT for anyone who edits this: the guard band (0.5 - 0.4999 = 1e-4) must stay above the
// largest error the fast quotient can have, which grows with the quotient: at |quotient| = 255 the
// reciprocal's one ulp plus the product's rounding come to about 4.6e-5.  Widening the code range
// (more than 8 bits) or replacing v_rcp_f32 by something less accurate needs a wider band; the
// known answers at 254.5 (tests/quantizer_kats.py, scale 3/256) and the tie stress in
// tests/test_gpu_cache.py fail if the band is too narrow.
template <int BITS>
__device__ __forceinline__ void codes8(const float (&w)[8], float scale, float bias, float inv, float (&q)[8]) {
    const float nb = (float)((1 << BITS) - 1);
    float dev = 0.0f;  // largest distance of a quotient from its rounded integer
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float r = __fmul_rn(__fsub_rn(w[j], bias), inv);
        const float c = rintf(r);
        dev = fmaxf(dev, fabsf(r - c));
        q[j] = fminf(fmaxf(c, 0.0f), nb);
    }
    if (dev > 0.4999f) {
#pragma unroll
        for (int j = 0; j < 8; ++j) q[j] = (float)affine_code(w[j], scale, bias, nb);
    }
}

// `v` of the lane whose number is byte_addr / 4
__device__ __forceinline__ float lane_value(int byte_addr, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(byte_addr, __builtin_bit_cast(int, v)));
}

// Four integer-valued floats in [0, 255] as the bytes of one word, first value lowest.
__device__ __forceinline__ uint32_t pack_bytes(float a, float b, float c, float d) {
    uint32_t w = __builtin_amdgcn_cvt_pk_u8_f32(a, 0, 0);
    w = __builtin_amdgcn_cvt_pk_u8_f32(b, 1, w);
    w = __builtin_amdgcn_cvt_pk_u8_f32(c, 2, w);
    return __builtin_amdgcn_cvt_pk_u8_f32(d, 3, w);
}
// Four integer-valued floats in [0, 15] as the nibbles of a 16-bit value, first value lowest
// (the sums stay below 2^16, so float32 arithmetic is exact).
__device__ __forceinline__ uint32_t pack_nibbles(float a, float b, float c, float d) {
    return (uint32_t)__builtin_fmaf(d, 4096.0f, __builtin_fmaf(c, 256.0f, __builtin_fmaf(b, 16.0f, a)));
}
// (scale, bias) of one group as the pair of 16-bit values the cache holds
template <int DT> __device__ __forceinline__ uint32_t pack_scale_bias(float scale, float bias) {
    if (DT == 0)
        return (uint32_t)__half_as_ushort(__float2half_rn(scale)) | ((uint32_t)__half_as_ushort(__float2half_rn(bias)) << 16);
    return (uint32_t)Elem<1>::bits(scale) | ((uint32_t)Elem<1>::bits(bias) << 16);
}

// grid (whole tiles, BH), 256 threads; slot0 is a multiple of 64; 16-bit dtypes, Dk == Dv == 32 NC;
// GL = group size / 8 lanes share a quantization group; ROPE = false carries no rotation code.
// A thread holds 16-byte chunks of K and of V rows (a "chunk-instance" each), up to eight at a
// time.  The extrema of every chunk-instance are reduced over the lanes of its group; then the
// affine parameters -- four exact divisions, the costly part -- are worked out once per group
// instead of once per lane: lane j of a group takes chunk-instance j (and j + GL, ...), writes
// that group's (scale, bias) pair, and the other lanes fetch bias and reciprocal from it.
// PAGED: the 64 rows are tile `l_t / 64` of the full-precision page store `src` (a cache being
// converted) instead of rows of dense arrays: K chunks are read from the interleaved tile where
// they lie, the V tile (stored by column) is turned back into rows through LDS.
// SIDE: 0 keys and values of one head size 32 NC; 1 the keys alone, 2 the values alone (caches whose keys and
// values differ in head size take one launch for each, NC being that side's).
template <int DT, int BITS, int NC, int GL, bool ROPE, bool PAGED, int SIDE = 0>
__device__ __forceinline__ void append_quant_tile_body(const Store &st, const Store &src, const char *keys, const char *values,
                                                       int L, int src0, int slot0, const RopeDev &rope) {
    constexpr int D = 32 * NC;
    constexpr int GS = 8 * GL;
    constexpr int TPR = D / 8;   // threads per row
    constexpr int VP = D + 8;    // byte pitch of a token's V codes in LDS
    constexpr bool DO_K = SIDE != 2, DO_V = SIDE != 1;
    // chunks per batch (a divisor of NC; one side alone: a count whose instances share out evenly over a group's lanes)
    constexpr int EB = SIDE == 0 ? (NC < 4 ? NC : 4) : (NC % 4 == 0 ? 4 : 2);
    static_assert(NC % EB == 0, "a batch holds a whole number of chunks");
    // chunk-instances per batch: both sides (chunk e0 + i / 2, K or V by i & 1), or one side's chunks e0 + i
    constexpr int NI = SIDE == 0 ? 2 * EB : EB;
    auto chunk_of = [](int i) { return SIDE == 0 ? i / 2 : i; };
    auto is_v = [](int i) { return SIDE == 0 ? (i & 1) != 0 : SIDE == 2; };
    constexpr int SH = GL < NI ? GL : NI;  // lanes of a group that work out parameters
    constexpr int PER = (NI + SH - 1) / SH;  // chunk-instances per such lane (D = 96: six over four lanes, two of them take two)
    // a row's TPR threads: where 256 is a multiple of TPR the rows of a thread's chunks are 256 / TPR apart and
    // its columns the same; at D = 96 (12 threads per row) row and column are worked out per chunk
    constexpr bool EVEN = 256 % TPR == 0;
    constexpr bool GEN = BITS != 4 && BITS != 8;  // 2, 3, 5, 6 bits: codes as a plain bit stream, K rows and V tile rows alike
    __shared__ __attribute__((aligned(8))) uint8_t vcodes[DO_V ? TILE * VP : 8];
    __shared__ __attribute__((aligned(16))) uint8_t kcodes[GEN && DO_K ? TILE * D * BITS / 8 : 16];  // the tile's K rows as stored
    __shared__ __attribute__((aligned(16))) uint8_t vstage[PAGED && DO_V ? TILE * D * 2 : 16];  // the source V tile as stored
    const int bh = blockIdx.y;
    const int slot_t = slot0 + blockIdx.x * TILE;
    const int l_t = src0 + blockIdx.x * TILE;
    const char *kbase = PAGED ? nullptr : keys + ((size_t)bh * L + l_t) * D * 2;
    const char *vbase = PAGED ? nullptr : values + ((size_t)bh * L + l_t) * D * 2;
    u4v kraw[NC], vraw[NC];
    if constexpr (PAGED) {
        const char *kt = k_cell_ptr(src, bh, l_t) + kfp_off(src, l_t, 0);   // tile start: [chunk][token][16 B]
        const char *vt = v_cell_ptr(src, bh, l_t) + vfp_off(src, l_t, 0);   // tile start: [8-token chunk][column][16 B]
#pragma unroll
        for (int e = 0; e < NC; ++e) {
            const int c = e * 256 + threadIdx.x;
            const int r = c / TPR, ch = c - r * TPR;
            if constexpr (DO_K) kraw[e] = *reinterpret_cast<const u4v *>(kt + ((size_t)ch * TILE + r) * 16);
            if constexpr (DO_V) *reinterpret_cast<u4v *>(vstage + (size_t)c * 16) = *reinterpret_cast<const u4v *>(vt + (size_t)c * 16);
        }
        if constexpr (DO_V) __syncthreads();
#pragma unroll
        for (int e = 0; e < (DO_V ? NC : 0); ++e) {
            const int c = e * 256 + threadIdx.x;
            const int r = c / TPR, dd = (c - r * TPR) * 8;
            const uint16_t *col = reinterpret_cast<const uint16_t *>(vstage) + ((size_t)(r >> 3) * D + dd) * 8 + (r & 7);
            uint32_t u[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) u[j] = (uint32_t)col[(2 * j) * 8] | ((uint32_t)col[(2 * j + 1) * 8] << 16);
            vraw[e] = u4v{u[0], u[1], u[2], u[3]};
        }
    } else {
#pragma unroll
        for (int e = 0; e < NC; ++e) {
            const int c = e * 256 + threadIdx.x;
            if constexpr (DO_K) kraw[e] = *reinterpret_cast<const u4v *>(kbase + (size_t)c * 16);
            if constexpr (DO_V) vraw[e] = *reinterpret_cast<const u4v *>(vbase + (size_t)c * 16);
        }
    }
    const RopeDev no_rope;
    const float nb = (float)((1 << BITS) - 1);
    const int lane = threadIdx.x & 63;
    const int pos = lane & (GL - 1);            // place in the group
    const int psel = pos & (SH - 1);
    const int gbase4 = (lane & ~(GL - 1)) * 4;  // byte address (lane number x 4) of the group's first lane
    const int r_t = threadIdx.x / TPR;          // row of this thread's chunk 0; chunk e lies 256 / TPR rows further
    const int d0_t = (threadIdx.x - r_t * TPR) * 8;
    auto row_of = [&](int e) { return EVEN ? r_t + e * (256 / TPR) : (e * 256 + (int)threadIdx.x) / TPR; };
    auto col_of = [&](int e) { return EVEN ? d0_t : ((e * 256 + (int)threadIdx.x) % TPR) * 8; };
    const int page_off = (slot_t & (PAGE - 1));
    const PageEntry page = st.pt[slot_t >> PAGE_SHIFT];  // a tile lies inside one page
#pragma unroll
    for (int e0 = 0; e0 < NC; e0 += EB) {
        float w[NI][8], mn[NI], mx[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int e = e0 + chunk_of(i);
            const int d0 = col_of(e);
            if (!is_v(i)) {
                const int r = row_of(e);
                if constexpr (ROPE) unpack8<DT>(kraw[e], kbase + (size_t)r * D * 2, d0, rope, rope_pos(rope, bh, l_t + r), w[i]);
                else unpack8<DT>(kraw[e], nullptr, d0, no_rope, 0, w[i]);
            } else {
                unpack8<DT>(vraw[e], nullptr, d0, no_rope, 0, w[i]);
            }
            float a = w[i][0], b = w[i][0];
#pragma unroll
            for (int j = 1; j < 8; ++j) {
                a = fminf(a, w[i][j]);
                b = fmaxf(b, w[i][j]);
            }
            group_minmax_dpp<GL>(a, b);
            mn[i] = a;
            mx[i] = b;
        }
        float sc[PER], bi[PER], iv[PER];
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            float a = mn[k * SH], b = mx[k * SH];
#pragma unroll
            for (int j = 1; j < SH; ++j)
                if (k * SH + j < NI) {
                    a = psel == j ? mn[k * SH + j] : a;
                    b = psel == j ? mx[k * SH + j] : b;
                }
            affine_params(a, b, nb, sc[k], bi[k]);
            iv[k] = __builtin_amdgcn_rcpf(sc[k]);
            if (pos < SH && psel + k * SH < NI) {
                const int i = psel + k * SH;  // this lane's chunk-instance
                const int row = page_off + row_of(e0 + chunk_of(i));
                const int d0 = col_of(e0 + chunk_of(i));
                char *sb = is_v(i) ? page.vsb + (size_t)bh * st.vsb_cell + (size_t)row * st.vsb_row
                                   : page.ksb + (size_t)bh * st.ksb_cell + (size_t)row * st.ksb_row;
                reinterpret_cast<uint32_t *>(sb)[d0 / GS] = pack_scale_bias<DT>(sc[k], bi[k]);
            }
        }
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int e = e0 + chunk_of(i);
            const int r = row_of(e), d0 = col_of(e);
            const int src = gbase4 + (i % SH) * 4;
            const float scale = lane_value(src, sc[i / SH]);
            const float bias = lane_value(src, bi[i / SH]);
            const float inv = lane_value(src, iv[i / SH]);
            float q[8];
            codes8<BITS>(w[i], scale, bias, inv, q);
            if (!is_v(i)) {
                // ---- K: packed words in natural order --------------------------------------------
                uint32_t *kw = reinterpret_cast<uint32_t *>(page.k + (size_t)bh * st.k_cell + (size_t)(page_off + r) * st.k_row);
                if constexpr (BITS == 4) {
                    kw[d0 / 8] = pack_nibbles(q[0], q[1], q[2], q[3]) | (pack_nibbles(q[4], q[5], q[6], q[7]) << 16);
                } else if constexpr (BITS == 8) {
                    *reinterpret_cast<uint2 *>(kw + d0 / 4) =
                        make_uint2(pack_bytes(q[0], q[1], q[2], q[3]), pack_bytes(q[4], q[5], q[6], q[7]));
                } else {
                    // eight codes are BITS whole bytes of the row's bit stream; the tile's K rows follow each other
                    // in the page, so they are collected in LDS and leave as 16-byte chunks below
                    uint64_t bits8 = 0;
#pragma unroll
                    for (int j = 0; j < 8; ++j) bits8 |= (uint64_t)(uint32_t)q[j] << (j * BITS);
                    uint8_t *kb = &kcodes[r * (D * BITS / 8) + (d0 / 8) * BITS];
#pragma unroll
                    for (int j = 0; j < BITS; ++j) kb[j] = (uint8_t)(bits8 >> (8 * j));
                }
            } else {
                // ---- V: codes as bytes, transposed below -----------------------------------------
                *reinterpret_cast<uint2 *>(&vcodes[r * VP + d0]) =
                    make_uint2(pack_bytes(q[0], q[1], q[2], q[3]), pack_bytes(q[4], q[5], q[6], q[7]));
            }
        }
    }
    if constexpr (GEN && DO_K) {
        __syncthreads();
        char *kt = page.k + (size_t)bh * st.k_cell + (size_t)page_off * st.k_row;  // 64 rows of D BITS / 8 bytes, contiguous
        for (int c = threadIdx.x; c < TILE * D * BITS / 8 / 16; c += 256)
            *reinterpret_cast<u4v *>(kt + (size_t)c * 16) = *reinterpret_cast<const u4v *>(&kcodes[c * 16]);
    }
    if constexpr (!DO_V) return;
    if constexpr (!(GEN && DO_K)) __syncthreads();
    char *cell = page.v + (size_t)bh * st.v_cell + v_row_off(st, slot_t, 0);
    if constexpr (GEN) {
        // a transposed row is the bit stream of its 64 tokens' codes, 2 BITS words: each thread assembles one word
        // from the codes that have bits in it; consecutive threads write consecutive words
        constexpr int WPR = 2 * BITS;
        for (int c = threadIdx.x; c < D * WPR; c += 256) {
            const int d = c / WPR, w = c - d * WPR;
            const int t0 = (32 * w) / BITS;  // the first token with bits in word w
            uint32_t word = 0;
#pragma unroll
            for (int i = 0; i < 32 / BITS + 2; ++i) {
                const int t = t0 + i;
                if (t < TILE && t * BITS < 32 * w + 32) word |= stream_bits(vcodes[t * VP + d], t * BITS, w);
            }
            reinterpret_cast<uint32_t *>(cell + (size_t)d * (TILE * BITS / 8))[w] = word;
        }
        return;
    }
    // each thread assembles 16 bytes (4 words) of one transposed row; consecutive threads
    // continue the same row, so the tile rows are written contiguously
    constexpr int TPW = 32 / BITS;        // tokens per word
    constexpr int CPR = TILE / TPW / 4;   // 16-byte chunks per row
    for (int c = threadIdx.x; c < D * CPR; c += 256) {
        const int d = c / CPR, q = c - d * CPR;
        uint32_t out[4];
#pragma unroll
        for (int wi = 0; wi < 4; ++wi) {
            uint32_t word = 0;
#pragma unroll
            for (int tt = 0; tt < TPW; ++tt) {
                const int t = (4 * q + wi) * TPW + tt;
                word |= (uint32_t)vcodes[t * VP + d] << (v_bitpos<BITS>(t) & 31);
            }
            out[wi] = word;
        }
        *reinterpret_cast<u4v *>(cell + (size_t)d * (TILE * BITS / 8) + 16 * q) = u4v{out[0], out[1], out[2], out[3]};
    }
}

template <int DT, int BITS, int NC, int GL, bool ROPE, int SIDE = 0>
__global__ void __launch_bounds__(256)
append_quant_tile_kernel(Store st, const char *keys, const char *values, int L, int src0, int slot0, RopeDev rope) {
    append_quant_tile_body<DT, BITS, NC, GL, ROPE, false, SIDE>(st, st, keys, values, L, src0, slot0, rope);
}

// grid (tiles, BH): tiles [0, gridDim.x) of the full-precision store `src` into the same slots of `st`
template <int DT, int BITS, int NC, int GL, int SIDE = 0>
__global__ void __launch_bounds__(256) requant_tile_kernel(Store st, Store src) {
    append_quant_tile_body<DT, BITS, NC, GL, false, true, SIDE>(st, src, nullptr, nullptr, 0, 0, 0, RopeDev());
}

// Which stores the tile kernels take: 16-bit dtypes, group size 32 / 64 / 128 dividing the head size; keys and
// values of one head size in 64 / 96 / 128 / 256 (one launch), or keys of 192 with values of 128 (a launch for
// each side; 4- and 8-bit codes, group size 32 or 64).
inline bool quant_tiles_one_launch(const Store &st) {
    return st.es == 2 && st.Dk == st.Dv && (st.Dk == 64 || st.Dk == 96 || st.Dk == 128 || st.Dk == 256) &&
           (st.gs == 32 || st.gs == 64 || st.gs == 128) && st.Dk % st.gs == 0;
}
inline bool quant_tiles_two_sided(const Store &st) {
    return st.es == 2 && st.Dk == 192 && st.Dv == 128 && (st.bits == 4 || st.bits == 8) && (st.gs == 32 || st.gs == 64);
}

// The launches of one code width.  PAGED = false: `tiles` whole tiles of the dense rows from row a0 on into the slots
// from b0 on (a multiple of 64); PAGED = true: tiles [0, tiles) of the full-precision store `src` into the same slots.
// TWO_SIDED: also the instances for keys of 192 with values of 128.
template <int DT, int BITS, int NC, int GL, int SIDE, bool PAGED>
void launch_quant_tile_instance(const Store &st, const Store &src, const void *keys, const void *values, int L, int a0,
                                int b0, int tiles, hipStream_t s, const RopeDev &r) {
    dim3 grid(tiles, st.BH), block(256);
    if constexpr (PAGED) {
        hipLaunchKernelGGL((requant_tile_kernel<DT, BITS, NC, GL, SIDE>), grid, block, 0, s, st, src);
    } else {
        if (r.dims > 0 && SIDE != 2)
            hipLaunchKernelGGL((append_quant_tile_kernel<DT, BITS, NC, GL, true, SIDE>), grid, block, 0, s, st,
                               (const char *)keys, (const char *)values, L, a0, b0, r);
        else
            hipLaunchKernelGGL((append_quant_tile_kernel<DT, BITS, NC, GL, false, SIDE>), grid, block, 0, s, st,
                               (const char *)keys, (const char *)values, L, a0, b0, r);
    }
}

template <int DT, int BITS, bool TWO_SIDED, bool PAGED>
hipError_t launch_quant_tiles_dt(const Store &st, const Store &src, const void *keys, const void *values, int L, int a0,
                                 int b0, int tiles, hipStream_t s, const RopeDev &r) {
#define KV_TILE(NC, GL, SIDE) launch_quant_tile_instance<DT, BITS, NC, GL, SIDE, PAGED>(st, src, keys, values, L, a0, b0, tiles, s, r)
#define KV_TILE_GL(NC)                        \
    do {                                      \
        if (st.gs == 32) KV_TILE(NC, 4, 0);   \
        else if (st.gs == 64) KV_TILE(NC, 8, 0); \
        else KV_TILE(NC, 16, 0);              \
    } while (0)
    if (quant_tiles_one_launch(st)) {
        if (st.Dk == 64) KV_TILE_GL(2);
        else if (st.Dk == 96) KV_TILE(3, 4, 0);
        else if (st.Dk == 128) KV_TILE_GL(4);
        else KV_TILE_GL(8);
        return hipGetLastError();
    }
    if constexpr (TWO_SIDED) {
        if (quant_tiles_two_sided(st)) {
            if (st.gs == 32) {
                KV_TILE(6, 4, 1);
                KV_TILE(4, 4, 2);
            } else {
                KV_TILE(6, 8, 1);
                KV_TILE(4, 8, 2);
            }
            return hipGetLastError();
        }
    }
#undef KV_TILE_GL
#undef KV_TILE
    return hipErrorInvalidValue;
}

template <int BITS, bool TWO_SIDED, bool PAGED>
hipError_t launch_quant_tiles_bits(const Store &st, const Store &src, const void *keys, const void *values, int L, int a0,
                                   int b0, int tiles, hipStream_t s, const RopeDev &r) {
    if (tiles <= 0) return hipSuccess;
    if (st.dtype == KVHIP_F16) return launch_quant_tiles_dt<0, BITS, TWO_SIDED, PAGED>(st, src, keys, values, L, a0, b0, tiles, s, r);
    if (st.dtype == KVHIP_BF16) return launch_quant_tiles_dt<1, BITS, TWO_SIDED, PAGED>(st, src, keys, values, L, a0, b0, tiles, s, r);
    return hipErrorInvalidValue;
}

}  // namespace

}  // namespace kvhip
