// Append (full precision and quantize-on-append), import/export between the
// page layout and the reference's dense array layout, ring-order gather, and
// the standalone affine quantizer.
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

// grid (L, B*H): one row per workgroup
template <int DT>
__global__ void rope_apply_kernel(RopeDev r, const char *x, char *out, int L, int D) {
    const int bh = blockIdx.y, l = blockIdx.x;
    const size_t off = ((size_t)bh * L + l) * D * (DT == 2 ? 4 : 2);
    const int pos = rope_pos(r, bh, l);
    // every element is read (with its partner) before any is written: out may alias x
    float v[4];
    int cnt = 0;
    for (int d = threadIdx.x; d < D; d += blockDim.x) v[cnt++] = rope_elem<DT>(r, x + off, d, pos);
    __syncthreads();
    cnt = 0;
    for (int d = threadIdx.x; d < D; d += blockDim.x) Elem<DT>::store(out + off, d, v[cnt++]);
}

// One wavefront quantizes one row of D elements.  Optional outputs:
//   k_words   packed codes in MLX order (D*BITS/32 words)
//   code_out  one byte per element (for the transposed V assembly)
//   sb_row    (scale,bias) pairs of dtype DT per group
//   scales/biases separate arrays of dtype DT per group
template <int DT, int BITS>
__device__ __forceinline__ void quantize_row_wave(const void *src, int D, int gs, int lane,
                                                  uint32_t *k_words, uint8_t *code_out, void *sb_row,
                                                  void *scales, void *biases, const RopeDev *rope = nullptr,
                                                  int pos = 0) {
    quantize_row_wave_from<DT, BITS>(
        [&](int d) { return rope ? rope_elem<DT>(*rope, src, d, pos) : Elem<DT>::load(src, d); }, D, gs, lane, k_words,
        [&](int d, uint32_t code) { if (code_out) code_out[d] = (uint8_t)code; }, sb_row, scales, biases);
}

// grid (rows, BH): one new row per workgroup, scattered into the chunk-interleaved tile.
template <int ES>
__global__ void append_fp_kernel(Store st, const char *keys, const char *values, int L, int src0,
                                 int slot0, RopeDev rope) {
    const int bh = blockIdx.y;
    const int i = blockIdx.x;
    const int slot = slot0 + i;
    const int l = src0 + i;
    using E = typename std::conditional<ES == 2, uint16_t, uint32_t>::type;
    const E *ks = reinterpret_cast<const E *>(keys) + ((size_t)bh * L + l) * st.Dk;
    char *kc = const_cast<char *>(k_cell_ptr(st, bh, slot));
    if (rope.dims > 0) {
        const int pos = rope_pos(rope, bh, l);
        for (int d = threadIdx.x; d < st.Dk; d += blockDim.x) {
            char *dst = kc + kfp_off(st, slot, d);
            if (ES == 4) Elem<2>::store(dst, 0, rope_elem<2>(rope, ks, d, pos));
            else if (st.dtype == KVHIP_F16) Elem<0>::store(dst, 0, rope_elem<0>(rope, ks, d, pos));
            else Elem<1>::store(dst, 0, rope_elem<1>(rope, ks, d, pos));
        }
    } else {
        for (int d = threadIdx.x; d < st.Dk; d += blockDim.x) *reinterpret_cast<E *>(kc + kfp_off(st, slot, d)) = ks[d];
    }
    const E *vs = reinterpret_cast<const E *>(values) + ((size_t)bh * L + l) * st.Dv;
    char *vc = const_cast<char *>(v_cell_ptr(st, bh, slot));
    for (int d = threadIdx.x; d < st.Dv; d += blockDim.x) *reinterpret_cast<E *>(vc + vfp_off(st, slot, d)) = vs[d];
}

// grid (64-token tiles touched, BH), 256 threads.  Each wavefront quantizes rows of
// the tile; V codes are staged as bytes in LDS and then merged into the transposed
// tile rows, touching only the token positions this append writes.
// (ROPE = false carries no rotation code: the single-token decode append stays as small as it was)
// PAGED: the new rows are rows [src0, src0 + n) of the full-precision page store `src` (a cache
// being converted) instead of dense arrays.
template <int DT, int BITS, bool ROPE, bool PAGED>
__device__ __forceinline__ void append_quant_body(const Store &st, const Store &src, const char *keys, const char *values,
                                                  int L, int src0, int slot0, int n, const RopeDev &rope) {
    extern __shared__ uint8_t vcodes[];  // [64][Dv]
    const int bh = blockIdx.y;
    const int tile = (slot0 >> 6) + blockIdx.x;
    const int lo = max(slot0, tile * TILE);
    const int hi = min(slot0 + n, tile * TILE + TILE);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    constexpr int TPW = 32 / BITS;          // tokens per word
    const int t_lo = lo & (TILE - 1), t_hi = t_lo + (hi - lo);
    // the words of a V tile row this append touches, and this thread's first merge item:
    // its old word is requested now, so a single-token append does not wait for it later
    // (for 3, 5 and 6 bits a token's code may straddle two words of the row's bit stream)
    const int w_lo = (t_lo * BITS) >> 5, nw = ((t_hi * BITS - 1) >> 5) - w_lo + 1;
    const int items = st.Dv * nw;
    char *cell = const_cast<char *>(v_cell_ptr(st, bh, lo));
    auto word_ptr = [&](int u) -> uint32_t * {
        const int d = u / nw, w = w_lo + (u - d * nw);
        return reinterpret_cast<uint32_t *>(cell + v_row_off(st, lo, d)) + w;
    };
    const bool partial = ((t_lo * BITS) & 31) != 0 || ((t_hi * BITS) & 31) != 0;  // some word keeps old tokens
    uint32_t old0 = 0;
    if (partial && (int)threadIdx.x < items) old0 = *word_ptr(threadIdx.x);
    // (row, K or V) pairs go round the wavefronts (four, or eight for appends of three rows and more), so one
    // new token uses two of them
    const int nwaves = blockDim.x >> 6;
    for (int item = wave; item < 2 * (hi - lo); item += nwaves) {
        const int slot = lo + (item >> 1);
        const int l = src0 + (slot - slot0);
        uint32_t *kw = reinterpret_cast<uint32_t *>(const_cast<char *>(k_row_ptr(st, bh, slot)));
        if constexpr (PAGED) {
            if ((item & 1) == 0) {
                const char *kc = k_cell_ptr(src, bh, l);
                quantize_row_wave_from<DT, BITS>([&](int d) { return Elem<DT>::load(kc + kfp_off(src, l, d), 0); }, st.Dk, st.gs,
                                                 lane, kw, [](int, uint32_t) {}, const_cast<char *>(ksb_row_ptr(st, bh, slot)),
                                                 nullptr, nullptr);
            } else {
                const char *vc = v_cell_ptr(src, bh, l);
                uint8_t *vc_out = vcodes + (slot & (TILE - 1)) * st.Dv;
                quantize_row_wave_from<DT, BITS>([&](int d) { return Elem<DT>::load(vc + vfp_off(src, l, d), 0); }, st.Dv, st.gs,
                                                 lane, nullptr, [&](int d, uint32_t code) { vc_out[d] = (uint8_t)code; },
                                                 const_cast<char *>(vsb_row_ptr(st, bh, slot)), nullptr, nullptr);
            }
        } else if ((item & 1) == 0) {
            const char *krow = keys + ((size_t)bh * L + l) * st.Dk * st.es;
            quantize_row_wave<DT, BITS>(krow, st.Dk, st.gs, lane, kw, nullptr, const_cast<char *>(ksb_row_ptr(st, bh, slot)),
                                        nullptr, nullptr, ROPE ? &rope : nullptr, ROPE ? rope_pos(rope, bh, l) : 0);
        } else {
            const char *vrow = values + ((size_t)bh * L + l) * st.Dv * st.es;
            quantize_row_wave<DT, BITS>(vrow, st.Dv, st.gs, lane, nullptr, vcodes + (slot & (TILE - 1)) * st.Dv,
                                        const_cast<char *>(vsb_row_ptr(st, bh, slot)), nullptr, nullptr);
        }
    }
    __syncthreads();
    for (int u = threadIdx.x; u < items; u += blockDim.x) {
        const int d = u / nw, w = w_lo + (u - d * nw);
        uint32_t nbits = 0, mbits = 0;
        if constexpr ((32 % BITS) == 0) {
            for (int tt = 0; tt < TPW; ++tt) {
                const int t = w * TPW + tt;
                if (t >= t_lo && t < t_hi) {
                    const int bp = v_bitpos<BITS>(t) & 31;
                    nbits |= (uint32_t)vcodes[t * st.Dv + d] << bp;
                    mbits |= ((1u << BITS) - 1u) << bp;
                }
            }
        } else {
            const int t0 = (32 * w) / BITS;  // the first token with bits in word w
            for (int tt = 0; tt < TPW + 2; ++tt) {
                const int t = t0 + tt;
                if (t >= t_lo && t < t_hi && t * BITS < 32 * w + 32) {
                    nbits |= stream_bits(vcodes[t * st.Dv + d], t * BITS, w);
                    mbits |= stream_bits((1u << BITS) - 1u, t * BITS, w);
                }
            }
        }
        uint32_t *p = word_ptr(u);
        if (mbits == 0xffffffffu) {
            *p = nbits;
        } else {
            const uint32_t old = (u == (int)threadIdx.x) ? old0 : *p;
            *p = (old & ~mbits) | nbits;
        }
    }
}

// grid (64-token tiles touched, BH), 256 threads.  Each wavefront quantizes rows of
// the tile; V codes are staged as bytes in LDS and then merged into the transposed
// tile rows, touching only the token positions this append writes.
// (ROPE = false carries no rotation code: the single-token decode append stays as small as it was)
template <int DT, int BITS, bool ROPE>
__global__ void __launch_bounds__(512)
append_quant_kernel(Store st, const char *keys, const char *values, int L, int src0, int slot0, int n,
                    RopeDev rope) {
    append_quant_body<DT, BITS, ROPE, false>(st, st, keys, values, L, src0, slot0, n, rope);
}

// The same for rows [row0, row0 + n) of a full-precision page store, written to the same slots of `st`.
template <int DT, int BITS>
__global__ void __launch_bounds__(256) requant_rows_kernel(Store st, Store src, int row0, int n) {
    append_quant_body<DT, BITS, false, true>(st, src, nullptr, nullptr, 0, row0, row0, n, RopeDev());
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

// v of the lane that the data-parallel-primitive control CTRL names (all lanes take part)
template <int CTRL> __device__ __forceinline__ float dpp_lane(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v),
                                                                 CTRL, 0xF, 0xF, false));
}

// Min/max over GL (4, 8 or 16) adjacent lanes without LDS round trips: two quad permutes, then
// the mirror of each half row and of each row (the lanes of a quad, then of a half row, already
// agree, so the mirrored lane holds the other half's result).  Minimum and maximum do not depend
// on the order of the reduction, so the values are those of group_minmax.
template <int GL> __device__ __forceinline__ void group_minmax_dpp(float &mn, float &mx) {
    mn = fminf(mn, dpp_lane<0xB1>(mn));  // quad_perm [1,0,3,2]
    mx = fmaxf(mx, dpp_lane<0xB1>(mx));
    mn = fminf(mn, dpp_lane<0x4E>(mn));  // quad_perm [2,3,0,1]
    mx = fmaxf(mx, dpp_lane<0x4E>(mx));
    if constexpr (GL >= 8) {
        mn = fminf(mn, dpp_lane<0x141>(mn));  // row_half_mirror
        mx = fmaxf(mx, dpp_lane<0x141>(mx));
    }
    if constexpr (GL >= 16) {
        mn = fminf(mn, dpp_lane<0x140>(mn));  // row_mirror
        mx = fmaxf(mx, dpp_lane<0x140>(mx));
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
    __shared__ __attribute__((aligned(8))) uint8_t vcodes[DO_V ? TILE * VP : 8];
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
                if (BITS == 4) {
                    kw[d0 / 8] = pack_nibbles(q[0], q[1], q[2], q[3]) | (pack_nibbles(q[4], q[5], q[6], q[7]) << 16);
                } else {
                    *reinterpret_cast<uint2 *>(kw + d0 / 4) =
                        make_uint2(pack_bytes(q[0], q[1], q[2], q[3]), pack_bytes(q[4], q[5], q[6], q[7]));
                }
            } else {
                // ---- V: codes as bytes, transposed below -----------------------------------------
                *reinterpret_cast<uint2 *>(&vcodes[r * VP + d0]) =
                    make_uint2(pack_bytes(q[0], q[1], q[2], q[3]), pack_bytes(q[4], q[5], q[6], q[7]));
            }
        }
    }
    if constexpr (!DO_V) return;
    __syncthreads();
    // each thread assembles 16 bytes (4 words) of one transposed row; consecutive threads
    // continue the same row, so the tile rows are written contiguously
    constexpr int TPW = 32 / BITS;        // tokens per word
    constexpr int CPR = TILE / TPW / 4;   // 16-byte chunks per row
    char *cell = page.v + (size_t)bh * st.v_cell + v_row_off(st, slot_t, 0);
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

// grid (64-token tiles, BH): rows [0, rows) of a quantized store as full-precision rows of `dst`
// (`MLX.dequantized`: scale * code + bias in float32, rounded once to the dtype)
template <int DT, int BITS>
__global__ void __launch_bounds__(256) dequant_pages_kernel(Store q, Store dst, int rows) {
    const int bh = blockIdx.y;
    const int lo = blockIdx.x * TILE, hi = min(rows, lo + TILE);
    for (int idx = threadIdx.x; idx < (hi - lo) * q.Dk; idx += 256) {
        const int t = idx / q.Dk, d = idx - t * q.Dk, slot = lo + t;
        const uint32_t c = stream_code<BITS>(reinterpret_cast<const uint32_t *>(k_row_ptr(q, bh, slot)), d);
        const char *sb = ksb_row_ptr(q, bh, slot);
        const float sc = Elem<DT>::load(sb, 2 * (d / q.gs)), bi = Elem<DT>::load(sb, 2 * (d / q.gs) + 1);
        Elem<DT>::store(const_cast<char *>(k_cell_ptr(dst, bh, slot)) + kfp_off(dst, slot, d), 0, __fadd_rn(__fmul_rn(sc, (float)c), bi));
    }
    const char *vcell = v_cell_ptr(q, bh, lo);
    for (int idx = threadIdx.x; idx < (hi - lo) * q.Dv; idx += 256) {
        const int d = idx / (hi - lo), t = idx - d * (hi - lo), slot = lo + t;   // consecutive threads: consecutive tokens of a column
        const uint32_t c = v_code_load<BITS>(vcell + v_row_off(q, lo, d), t);
        const char *sb = vsb_row_ptr(q, bh, slot);
        const float sc = Elem<DT>::load(sb, 2 * (d / q.gs)), bi = Elem<DT>::load(sb, 2 * (d / q.gs) + 1);
        Elem<DT>::store(const_cast<char *>(v_cell_ptr(dst, bh, slot)) + vfp_off(dst, slot, d), 0, __fadd_rn(__fmul_rn(sc, (float)c), bi));
    }
}

// grid (whole tiles, BH), 256 threads; 16-bit dtypes, Dk == 32 NCK, Dv == 32 NCV
template <int NCK, int NCV>
__global__ void __launch_bounds__(256)
append_fp_tile_kernel(Store st, const char *keys, const char *values, int L, int src0, int slot0, RopeDev rope) {
    constexpr int DK = 32 * NCK, D = 32 * NCV;
    constexpr int TPRK = DK / 8, TPR = D / 8;
    constexpr int VPW = D / 2 + 1;  // dword pitch of a token's V row in LDS (odd: column reads spread over banks)
    __shared__ uint32_t vt[TILE * VPW];
    const int bh = blockIdx.y;
    const int slot_t = slot0 + blockIdx.x * TILE;
    const int l_t = src0 + blockIdx.x * TILE;
    const char *kbase = keys + ((size_t)bh * L + l_t) * DK * 2;
    const char *vbase = values + ((size_t)bh * L + l_t) * D * 2;
    char *kcell = st.pt[slot_t >> PAGE_SHIFT].k + (size_t)bh * st.k_cell;  // a tile lies inside one page
    u4v kraw[NCK], vraw[NCV];
#pragma unroll
    for (int e = 0; e < NCK; ++e) kraw[e] = *reinterpret_cast<const u4v *>(kbase + (size_t)(e * 256 + threadIdx.x) * 16);
#pragma unroll
    for (int e = 0; e < NCV; ++e) vraw[e] = *reinterpret_cast<const u4v *>(vbase + (size_t)(e * 256 + threadIdx.x) * 16);
#pragma unroll
    for (int e = 0; e < NCK; ++e) {
        const int c = e * 256 + threadIdx.x;
        const int r = c / TPRK, d0 = (c - r * TPRK) * 8;
        u4v k = kraw[e];
        if (rope.dims > 0 && d0 < rope.dims) {
            const int pos = rope_pos(rope, bh, l_t + r);
            const char *row = kbase + (size_t)r * DK * 2;
            uint32_t u[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint16_t lo, hi;
                if (st.dtype == KVHIP_F16) {
                    lo = __half_as_ushort(__float2half_rn(rope_elem<0>(rope, row, d0 + 2 * j, pos)));
                    hi = __half_as_ushort(__float2half_rn(rope_elem<0>(rope, row, d0 + 2 * j + 1, pos)));
                } else {
                    lo = Elem<1>::bits(rope_elem<1>(rope, row, d0 + 2 * j, pos));
                    hi = Elem<1>::bits(rope_elem<1>(rope, row, d0 + 2 * j + 1, pos));
                }
                u[j] = (uint32_t)lo | ((uint32_t)hi << 16);
            }
            k = u4v{u[0], u[1], u[2], u[3]};
        }
        *reinterpret_cast<u4v *>(kcell + kfp_off(st, slot_t + r, d0)) = k;
    }
#pragma unroll
    for (int e = 0; e < NCV; ++e) {
        const int c = e * 256 + threadIdx.x;
        const int r = c / TPR, d0 = (c - r * TPR) * 8;
        uint32_t *vrow = &vt[r * VPW + d0 / 2];
        vrow[0] = vraw[e].x;
        vrow[1] = vraw[e].y;
        vrow[2] = vraw[e].z;
        vrow[3] = vraw[e].w;
    }
    __syncthreads();
    // 8-token chunks of every column: thread (c8, d) gathers tokens 8 c8 .. 8 c8 + 7 of column d;
    // consecutive threads take consecutive columns, so a chunk row is written contiguously
    char *cell = const_cast<char *>(v_cell_ptr(st, bh, slot_t));
    const uint16_t *vt16 = reinterpret_cast<const uint16_t *>(vt);
    for (int c = threadIdx.x; c < D * 8; c += 256) {
        const int c8 = c / D, d = c - c8 * D;
        uint32_t out[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo = vt16[(8 * c8 + 2 * j) * (2 * VPW) + d];
            const uint32_t hi = vt16[(8 * c8 + 2 * j + 1) * (2 * VPW) + d];
            out[j] = lo | (hi << 16);
        }
        *reinterpret_cast<u4v *>(cell + vfp_off(st, slot_t + 8 * c8, d)) = u4v{out[0], out[1], out[2], out[3]};
    }
}

template <int ES>
__global__ void export_fp_kernel(Store st, Runs runs, int row_begin, int dst_row0, int nrows, char *dst_k, char *dst_v) {
    const int bh = blockIdx.y;
    const int slot = row_to_slot(runs, row_begin + blockIdx.x);
    const int i = row_begin + blockIdx.x - dst_row0;  // row of the dense destination [BH, nrows, D]
    if (slot < 0) return;
    using E = typename std::conditional<ES == 2, uint16_t, uint32_t>::type;
    if (dst_k) {
        const char *kc = k_cell_ptr(st, bh, slot);
        E *kd = reinterpret_cast<E *>(dst_k) + ((size_t)bh * nrows + i) * st.Dk;
        for (int d = threadIdx.x; d < st.Dk; d += blockDim.x) kd[d] = *reinterpret_cast<const E *>(kc + kfp_off(st, slot, d));
    }
    if (dst_v) {
        const char *vc = v_cell_ptr(st, bh, slot);
        E *vd = reinterpret_cast<E *>(dst_v) + ((size_t)bh * nrows + i) * st.Dv;
        for (int d = threadIdx.x; d < st.Dv; d += blockDim.x)
            vd[d] = *reinterpret_cast<const E *>(vc + vfp_off(st, slot, d));
    }
}

template <int ES>
__global__ void import_fp_kernel(Store st, const char *src_k, const char *src_v, int nrows) {
    const int bh = blockIdx.y;
    const int slot = blockIdx.x;
    using E = typename std::conditional<ES == 2, uint16_t, uint32_t>::type;
    const E *ks = reinterpret_cast<const E *>(src_k) + ((size_t)bh * nrows + slot) * st.Dk;
    char *kc = const_cast<char *>(k_cell_ptr(st, bh, slot));
    for (int d = threadIdx.x; d < st.Dk; d += blockDim.x) *reinterpret_cast<E *>(kc + kfp_off(st, slot, d)) = ks[d];
    const E *vs = reinterpret_cast<const E *>(src_v) + ((size_t)bh * nrows + slot) * st.Dv;
    char *vc = const_cast<char *>(v_cell_ptr(st, bh, slot));
    for (int d = threadIdx.x; d < st.Dv; d += blockDim.x) *reinterpret_cast<E *>(vc + vfp_off(st, slot, d)) = vs[d];
}

template <int ES>
__global__ void compact_fp_kernel(Store src, Runs runs, Store dst, int nrows) {
    const int bh = blockIdx.y;
    const int i = blockIdx.x;
    const int slot = row_to_slot(runs, i);
    if (slot < 0) return;
    using E = typename std::conditional<ES == 2, uint16_t, uint32_t>::type;
    const char *ks = k_cell_ptr(src, bh, slot);
    char *kd = const_cast<char *>(k_cell_ptr(dst, bh, i));
    for (int d = threadIdx.x; d < src.Dk; d += blockDim.x)
        *reinterpret_cast<E *>(kd + kfp_off(dst, i, d)) = *reinterpret_cast<const E *>(ks + kfp_off(src, slot, d));
    const char *vs = v_cell_ptr(src, bh, slot);
    char *vd = const_cast<char *>(v_cell_ptr(dst, bh, i));
    for (int d = threadIdx.x; d < src.Dv; d += blockDim.x)
        *reinterpret_cast<E *>(vd + vfp_off(dst, i, d)) = *reinterpret_cast<const E *>(vs + vfp_off(src, slot, d));
}

// which: 0 k.wq 1 k.scales 2 k.biases 3 v.wq 4 v.scales 5 v.biases; grid (nrows, BH)
template <int BITS>
__global__ void export_quant_kernel(Store st, int which, int nrows, char *dst) {
    const int bh = blockIdx.y;
    const int slot = blockIdx.x;
    const int es = st.es;
    if (which == 0) {
        const int W = st.Dk * BITS / 32;
        const uint32_t *s = reinterpret_cast<const uint32_t *>(k_row_ptr(st, bh, slot));
        uint32_t *d = reinterpret_cast<uint32_t *>(dst) + ((size_t)bh * nrows + slot) * W;
        for (int w = threadIdx.x; w < W; w += blockDim.x) d[w] = s[w];
    } else if (which == 3) {
        constexpr int per = 32 / BITS;
        const int W = st.Dv * BITS / 32;
        const char *cell = v_cell_ptr(st, bh, slot);
        const int t = slot & (TILE - 1);
        uint32_t *d = reinterpret_cast<uint32_t *>(dst) + ((size_t)bh * nrows + slot) * W;
        for (int w = threadIdx.x; w < W; w += blockDim.x) {
            uint32_t word = 0;
            if constexpr ((32 % BITS) == 0) {
                for (int i = 0; i < per; ++i)
                    word |= v_code_load<BITS>(cell + v_row_off(st, slot, w * per + i), t) << (i * BITS);
            } else {
                const int j0 = (32 * w) / BITS;  // the first column with bits in word w of the row's bit stream
                for (int i = 0; i < per + 2; ++i) {
                    const int j = j0 + i;
                    if (j < st.Dv && j * BITS < 32 * w + 32)
                        word |= stream_bits(v_code_load<BITS>(cell + v_row_off(st, slot, j), t), j * BITS, w);
                }
            }
            d[w] = word;
        }
    } else {
        const bool isk = which < 3;
        const int G = (isk ? st.Dk : st.Dv) / st.gs;
        const int comp = (which == 1 || which == 4) ? 0 : 1;
        const char *s = isk ? ksb_row_ptr(st, bh, slot) : vsb_row_ptr(st, bh, slot);
        char *d = dst + ((size_t)bh * nrows + slot) * G * es;
        for (int g = threadIdx.x; g < G; g += blockDim.x) {
            if (es == 2)
                reinterpret_cast<uint16_t *>(d)[g] = reinterpret_cast<const uint16_t *>(s)[2 * g + comp];
            else
                reinterpret_cast<uint32_t *>(d)[g] = reinterpret_cast<const uint32_t *>(s)[2 * g + comp];
        }
    }
}

// grid (64-token tiles, BH): dense reference arrays into slots [0, nrows)
template <int BITS>
__global__ void import_quant_kernel(Store st, const uint32_t *kw, const char *ks, const char *kb,
                                    const uint32_t *vw, const char *vs, const char *vb, int nrows) {
    const int bh = blockIdx.y;
    const int lo = blockIdx.x * TILE, hi = min(nrows, lo + TILE);
    const int es = st.es;
    const int Wk = st.Dk * BITS / 32, Wv = st.Dv * BITS / 32, Gk = st.Dk / st.gs, Gv = st.Dv / st.gs;
    for (int slot = lo; slot < hi; ++slot) {
        const size_t r = (size_t)bh * nrows + slot;
        uint32_t *kd = reinterpret_cast<uint32_t *>(const_cast<char *>(k_row_ptr(st, bh, slot)));
        for (int w = threadIdx.x; w < Wk; w += blockDim.x) kd[w] = kw[r * Wk + w];
        char *ksd = const_cast<char *>(ksb_row_ptr(st, bh, slot));
        char *vsd = const_cast<char *>(vsb_row_ptr(st, bh, slot));
        for (int g = threadIdx.x; g < Gk; g += blockDim.x) {
            if (es == 2) {
                reinterpret_cast<uint16_t *>(ksd)[2 * g] = reinterpret_cast<const uint16_t *>(ks)[r * Gk + g];
                reinterpret_cast<uint16_t *>(ksd)[2 * g + 1] = reinterpret_cast<const uint16_t *>(kb)[r * Gk + g];
            } else {
                reinterpret_cast<uint32_t *>(ksd)[2 * g] = reinterpret_cast<const uint32_t *>(ks)[r * Gk + g];
                reinterpret_cast<uint32_t *>(ksd)[2 * g + 1] = reinterpret_cast<const uint32_t *>(kb)[r * Gk + g];
            }
        }
        for (int g = threadIdx.x; g < Gv; g += blockDim.x) {
            if (es == 2) {
                reinterpret_cast<uint16_t *>(vsd)[2 * g] = reinterpret_cast<const uint16_t *>(vs)[r * Gv + g];
                reinterpret_cast<uint16_t *>(vsd)[2 * g + 1] = reinterpret_cast<const uint16_t *>(vb)[r * Gv + g];
            } else {
                reinterpret_cast<uint32_t *>(vsd)[2 * g] = reinterpret_cast<const uint32_t *>(vs)[r * Gv + g];
                reinterpret_cast<uint32_t *>(vsd)[2 * g + 1] = reinterpret_cast<const uint32_t *>(vb)[r * Gv + g];
            }
        }
    }
    char *cell = const_cast<char *>(v_cell_ptr(st, bh, lo));
    constexpr int TPW = 32 / BITS;
    constexpr int WPR = TILE * BITS / 32;
    for (int u = threadIdx.x; u < st.Dv * WPR; u += blockDim.x) {
        const int d = u / WPR, w = u - d * WPR;
        uint32_t nbits = 0;
        if constexpr ((32 % BITS) == 0) {
            for (int tt = 0; tt < TPW; ++tt) {
                const int t = w * TPW + tt;
                if (lo + t < hi)
                    nbits |= stream_code<BITS>(vw + ((size_t)bh * nrows + lo + t) * Wv, d) << (v_bitpos<BITS>(t) & 31);
            }
        } else {
            const int t0 = (32 * w) / BITS;  // the first token with bits in word w of the tile row
            for (int tt = 0; tt < TPW + 2; ++tt) {
                const int t = t0 + tt;
                if (t < TILE && lo + t < hi && t * BITS < 32 * w + 32)
                    nbits |= stream_bits(stream_code<BITS>(vw + ((size_t)bh * nrows + lo + t) * Wv, d), t * BITS, w);
            }
        }
        reinterpret_cast<uint32_t *>(cell + v_row_off(st, lo, d))[w] = nbits;
    }
}

// one wavefront per row; grid.x * 4 waves
template <int DT, int BITS>
__global__ void __launch_bounds__(256)
affine_quantize_kernel(const char *src, int64_t rows, int D, int gs, uint32_t *wq, char *scales, char *biases, int es) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int W = D * BITS / 32, G = D / gs;
    quantize_row_wave<DT, BITS>(src + row * D * es, D, gs, lane, wq + row * W, nullptr, nullptr,
                                scales + row * G * es, biases + row * G * es);
}

template <int DT, int BITS>
__global__ void affine_dequantize_kernel(const uint32_t *wq, const char *scales, const char *biases,
                                         int64_t rows, int D, int gs, char *dst) {
    const int64_t row = blockIdx.x;
    const int W = D * BITS / 32, G = D / gs;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        const uint32_t c = stream_code<BITS>(wq + row * W, d);
        const float s = Elem<DT>::load(scales, row * G + d / gs);
        const float b = Elem<DT>::load(biases, row * G + d / gs);
        Elem<DT>::store(dst, row * D + d, __fadd_rn(__fmul_rn(s, (float)c), b));
    }
}

__global__ void mask_materialize_kernel(kvhip_mask_plan_t p, uint8_t *dst) {
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= p.cols) return;
    if (p.rolled) {
        // (arange(cols) >= cols - window) rolled right by roll_shift
        const int src = ((j - p.roll_shift) % p.cols + p.cols) % p.cols;
        dst[j] = src >= p.cols - p.roll_window;
        return;
    }
    for (int i = blockIdx.y; i < p.rows; i += gridDim.y) {
        const int li = p.offset + i;
        bool keep = li >= j;
        if (p.window > 0) keep = keep && (li < j + p.window);
        dst[(size_t)i * p.cols + j] = keep;
    }
}

}  // namespace

#define KV_DISPATCH_DT_BITS(DTV, BITSV, CALL)                                                  \
    do {                                                                                       \
        if ((BITSV) == 4) { if ((DTV) == 0) { CALL(0, 4); } else if ((DTV) == 1) { CALL(1, 4); } else { CALL(2, 4); } } \
        else if ((BITSV) == 8) { if ((DTV) == 0) { CALL(0, 8); } else if ((DTV) == 1) { CALL(1, 8); } else { CALL(2, 8); } } \
        else if ((BITSV) == 3) { if ((DTV) == 0) { CALL(0, 3); } else if ((DTV) == 1) { CALL(1, 3); } else { CALL(2, 3); } } \
        else if ((BITSV) == 5) { if ((DTV) == 0) { CALL(0, 5); } else if ((DTV) == 1) { CALL(1, 5); } else { CALL(2, 5); } } \
        else if ((BITSV) == 6) { if ((DTV) == 0) { CALL(0, 6); } else if ((DTV) == 1) { CALL(1, 6); } else { CALL(2, 6); } } \
        else { if ((DTV) == 0) { CALL(0, 2); } else if ((DTV) == 1) { CALL(1, 2); } else { CALL(2, 2); } } \
    } while (0)

namespace {
hipError_t launch_append_fp_rows(const Store &st, const void *keys, const void *values, int L, int src0,
                                 int slot0, int n, hipStream_t s, const RopeDev &r) {
    if (n <= 0) return hipSuccess;
    dim3 grid(n, st.BH), block(128);
    if (st.es == 2)
        hipLaunchKernelGGL(append_fp_kernel<2>, grid, block, 0, s, st, (const char *)keys, (const char *)values, L, src0, slot0, r);
    else
        hipLaunchKernelGGL(append_fp_kernel<4>, grid, block, 0, s, st, (const char *)keys, (const char *)values, L, src0, slot0, r);
    return hipGetLastError();
}
// slots [slot0, slot0 + n) as: rows up to the next tile boundary, whole tiles, remaining rows
struct TileSplit {
    int head, tiles, tail;
};
TileSplit tile_split(int slot0, int n) {
    TileSplit t{0, 0, 0};
    t.head = std::min(n, (TILE - (slot0 & (TILE - 1))) & (TILE - 1));
    t.tiles = (n - t.head) / TILE;
    t.tail = n - t.head - t.tiles * TILE;
    return t;
}
}  // namespace

hipError_t launch_append_fp(const Store &st, const void *keys, const void *values, int L, int src0,
                            int slot0, int n, hipStream_t s, const RopeDev *rope) {
    if (n <= 0) return hipSuccess;
    const RopeDev r = rope ? *rope : RopeDev();
    const bool mla = st.Dk == 192 && st.Dv == 128;  // keys of 192 with values of 128
    const bool tiled = st.es == 2 && ((st.Dk == st.Dv && (st.Dk == 64 || st.Dk == 96 || st.Dk == 128 || st.Dk == 256)) || mla);
    const TileSplit t = tile_split(slot0, n);
    if (!tiled || t.tiles == 0) return launch_append_fp_rows(st, keys, values, L, src0, slot0, n, s, r);
    hipError_t e = launch_append_fp_rows(st, keys, values, L, src0, slot0, t.head, s, r);
    if (e != hipSuccess) return e;
    dim3 grid(t.tiles, st.BH), block(256);
    const int a0 = src0 + t.head, b0 = slot0 + t.head;
#define FP_TILE(NCK, NCV) hipLaunchKernelGGL((append_fp_tile_kernel<NCK, NCV>), grid, block, 0, s, st, (const char *)keys, (const char *)values, L, a0, b0, r)
    if (mla) FP_TILE(6, 4);
    else if (st.Dk == 64) FP_TILE(2, 2);
    else if (st.Dk == 96) FP_TILE(3, 3);
    else if (st.Dk == 128) FP_TILE(4, 4);
    else FP_TILE(8, 8);
#undef FP_TILE
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_append_fp_rows(st, keys, values, L, a0 + t.tiles * TILE, b0 + t.tiles * TILE, t.tail, s, r);
}

hipError_t launch_rope_apply(const RopeDev &rope, const void *x, void *out, int B, int H, int L, int D,
                             int dtype, hipStream_t s) {
    if ((size_t)B * H * L == 0) return hipSuccess;
    dim3 grid(L, B * H), block(D <= 64 ? 64 : (D <= 128 ? 128 : 256));  // at most 4 elements per thread up to D = 1024
    if (dtype == KVHIP_F16) hipLaunchKernelGGL(rope_apply_kernel<0>, grid, block, 0, s, rope, (const char *)x, (char *)out, L, D);
    else if (dtype == KVHIP_BF16) hipLaunchKernelGGL(rope_apply_kernel<1>, grid, block, 0, s, rope, (const char *)x, (char *)out, L, D);
    else hipLaunchKernelGGL(rope_apply_kernel<2>, grid, block, 0, s, rope, (const char *)x, (char *)out, L, D);
    return hipGetLastError();
}

namespace {
hipError_t launch_append_quant_rows(const Store &st, const void *keys, const void *values, int L, int src0,
                                    int slot0, int n, hipStream_t s, const RopeDev &r) {
    if (n <= 0) return hipSuccess;
    const int ntile = ((slot0 + n - 1) >> 6) - (slot0 >> 6) + 1;
    // (a speculative-verify step appends 4 rows: 8 (row, K or V) items, one per wavefront)
    dim3 grid(ntile, st.BH), block(n >= 3 ? 512 : 256);
    const size_t lds = (size_t)TILE * st.Dv;
#define CALL(DT, BITS)                                                                                      \
    do {                                                                                                    \
        if (r.dims > 0)                                                                                     \
            hipLaunchKernelGGL((append_quant_kernel<DT, BITS, true>), grid, block, lds, s, st, (const char *)keys,  \
                               (const char *)values, L, src0, slot0, n, r);                                 \
        else                                                                                                \
            hipLaunchKernelGGL((append_quant_kernel<DT, BITS, false>), grid, block, lds, s, st, (const char *)keys, \
                               (const char *)values, L, src0, slot0, n, r);                                 \
    } while (0)
    KV_DISPATCH_DT_BITS(st.dtype, st.bits, CALL);
#undef CALL
    return hipGetLastError();
}
}  // namespace

hipError_t launch_append_quant(const Store &st, const void *keys, const void *values, int L, int src0,
                               int slot0, int n, hipStream_t s, const RopeDev *rope) {
    if (n <= 0) return hipSuccess;
    const RopeDev r = rope ? *rope : RopeDev();
    const bool tiled = st.es == 2 && st.Dk == st.Dv && (st.Dk == 64 || st.Dk == 96 || st.Dk == 128 || st.Dk == 256) &&
                       (st.bits == 4 || st.bits == 8) && (st.gs == 32 || st.gs == 64 || st.gs == 128) &&
                       st.Dk % st.gs == 0;
    // keys of 192 with values of 128: a launch for the keys and one for the values
    const bool two_sided = st.es == 2 && st.Dk == 192 && st.Dv == 128 && (st.bits == 4 || st.bits == 8) && (st.gs == 32 || st.gs == 64);
    const TileSplit t = tile_split(slot0, n);
    if ((!tiled && !two_sided) || t.tiles == 0) return launch_append_quant_rows(st, keys, values, L, src0, slot0, n, s, r);
    hipError_t e = launch_append_quant_rows(st, keys, values, L, src0, slot0, t.head, s, r);
    if (e != hipSuccess) return e;
    dim3 grid(t.tiles, st.BH), block(256);
    const int a0 = src0 + t.head, b0 = slot0 + t.head;
    if (two_sided) {
#define SIDE_CALL(DT, BITS, NC, GL, RP, SIDE)                                                                          \
    hipLaunchKernelGGL((append_quant_tile_kernel<DT, BITS, NC, GL, RP, SIDE>), grid, block, 0, s, st, (const char *)keys, \
                       (const char *)values, L, a0, b0, r)
#define SIDES(DT, BITS, GL)                                    \
    do {                                                       \
        if (r.dims > 0) SIDE_CALL(DT, BITS, 6, GL, true, 1);   \
        else SIDE_CALL(DT, BITS, 6, GL, false, 1);             \
        SIDE_CALL(DT, BITS, 4, GL, false, 2);                  \
    } while (0)
#define SIDES_GL(DT, BITS)                     \
    do {                                       \
        if (st.gs == 32) SIDES(DT, BITS, 4);   \
        else SIDES(DT, BITS, 8);               \
    } while (0)
        if (st.dtype == KVHIP_F16) {
            if (st.bits == 4) SIDES_GL(0, 4); else SIDES_GL(0, 8);
        } else {
            if (st.bits == 4) SIDES_GL(1, 4); else SIDES_GL(1, 8);
        }
#undef SIDES_GL
#undef SIDES
#undef SIDE_CALL
        e = hipGetLastError();
        if (e != hipSuccess) return e;
        return launch_append_quant_rows(st, keys, values, L, a0 + t.tiles * TILE, b0 + t.tiles * TILE, t.tail, s, r);
    }
#define TILE_CALL(DT, BITS, NC, GL, RP)                                                                  \
    hipLaunchKernelGGL((append_quant_tile_kernel<DT, BITS, NC, GL, RP>), grid, block, 0, s, st, (const char *)keys, \
                       (const char *)values, L, a0, b0, r)
#define TILE_RP(DT, BITS, NC, GL)                           \
    do {                                                    \
        if (r.dims > 0) TILE_CALL(DT, BITS, NC, GL, true);  \
        else TILE_CALL(DT, BITS, NC, GL, false);            \
    } while (0)
#define TILE_GL(DT, BITS, NC)                               \
    do {                                                    \
        if (st.gs == 32) TILE_RP(DT, BITS, NC, 4);          \
        else if (st.gs == 64) TILE_RP(DT, BITS, NC, 8);     \
        else TILE_RP(DT, BITS, NC, 16);                     \
    } while (0)
#define TILE_NC(DT, BITS)                              \
    do {                                               \
        if (st.Dk == 64) TILE_GL(DT, BITS, 2);         \
        else if (st.Dk == 96) TILE_RP(DT, BITS, 3, 4); \
        else if (st.Dk == 128) TILE_GL(DT, BITS, 4);   \
        else TILE_GL(DT, BITS, 8);                     \
    } while (0)
    if (st.dtype == KVHIP_F16) {
        if (st.bits == 4) TILE_NC(0, 4); else TILE_NC(0, 8);
    } else {
        if (st.bits == 4) TILE_NC(1, 4); else TILE_NC(1, 8);
    }
#undef TILE_NC
#undef TILE_GL
#undef TILE_RP
#undef TILE_CALL
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_append_quant_rows(st, keys, values, L, a0 + t.tiles * TILE, b0 + t.tiles * TILE, t.tail, s, r);
}

hipError_t launch_requant_pages(const Store &src, const Store &st, int rows, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    const int tiles = (rows + TILE - 1) / TILE;
    const bool tiled = st.es == 2 && st.Dk == st.Dv && (st.Dk == 64 || st.Dk == 96 || st.Dk == 128 || st.Dk == 256) &&
                       (st.bits == 4 || st.bits == 8) && (st.gs == 32 || st.gs == 64 || st.gs == 128) && st.Dk % st.gs == 0;
    dim3 grid(tiles, st.BH), block(256);
    if (st.es == 2 && st.Dk == 192 && st.Dv == 128 && (st.bits == 4 || st.bits == 8) && (st.gs == 32 || st.gs == 64)) {
        // keys of 192 with values of 128: a launch for the keys and one for the values
#define RQS(DT, BITS, GL)                                                                                      \
    do {                                                                                                       \
        hipLaunchKernelGGL((requant_tile_kernel<DT, BITS, 6, GL, 1>), grid, block, 0, s, st, src);             \
        hipLaunchKernelGGL((requant_tile_kernel<DT, BITS, 4, GL, 2>), grid, block, 0, s, st, src);             \
    } while (0)
#define RQS_GL(DT, BITS)                     \
    do {                                     \
        if (st.gs == 32) RQS(DT, BITS, 4);   \
        else RQS(DT, BITS, 8);               \
    } while (0)
        if (st.dtype == KVHIP_F16) {
            if (st.bits == 4) RQS_GL(0, 4); else RQS_GL(0, 8);
        } else {
            if (st.bits == 4) RQS_GL(1, 4); else RQS_GL(1, 8);
        }
#undef RQS_GL
#undef RQS
        return hipGetLastError();
    }
    if (!tiled) {
        const size_t lds = (size_t)TILE * st.Dv;
#define CALL(DT, BITS) hipLaunchKernelGGL((requant_rows_kernel<DT, BITS>), grid, block, lds, s, st, src, 0, rows)
        KV_DISPATCH_DT_BITS(st.dtype, st.bits, CALL);
#undef CALL
        return hipGetLastError();
    }
    // whole tiles, the last one included: its rows past `rows` hold zeros or rows trimmed earlier, and
    // what they quantize to lies past the new cache's offset, where the next append overwrites it
#define RQ(DT, BITS, NC, GL) hipLaunchKernelGGL((requant_tile_kernel<DT, BITS, NC, GL>), grid, block, 0, s, st, src)
#define RQ_GL(DT, BITS, NC)                            \
    do {                                               \
        if (st.gs == 32) RQ(DT, BITS, NC, 4);          \
        else if (st.gs == 64) RQ(DT, BITS, NC, 8);     \
        else RQ(DT, BITS, NC, 16);                     \
    } while (0)
#define RQ_NC(DT, BITS)                              \
    do {                                             \
        if (st.Dk == 64) RQ_GL(DT, BITS, 2);         \
        else if (st.Dk == 96) RQ(DT, BITS, 3, 4);    \
        else if (st.Dk == 128) RQ_GL(DT, BITS, 4);   \
        else RQ_GL(DT, BITS, 8);                     \
    } while (0)
    if (st.dtype == KVHIP_F16) {
        if (st.bits == 4) RQ_NC(0, 4); else RQ_NC(0, 8);
    } else {
        if (st.bits == 4) RQ_NC(1, 4); else RQ_NC(1, 8);
    }
#undef RQ_NC
#undef RQ_GL
#undef RQ
    return hipGetLastError();
}

hipError_t launch_dequant_pages(const Store &q, const Store &dst, int rows, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    dim3 grid((rows + TILE - 1) / TILE, q.BH), block(256);
#define CALL(DT, BITS) hipLaunchKernelGGL((dequant_pages_kernel<DT, BITS>), grid, block, 0, s, q, dst, rows)
    KV_DISPATCH_DT_BITS(q.dtype, q.bits, CALL);
#undef CALL
    return hipGetLastError();
}

hipError_t launch_export_fp(const Store &st, const Runs &runs, int row_begin, int count, int dst_row0,
                            int dst_rows, void *dst_k, void *dst_v, hipStream_t s) {
    if (count <= 0) return hipSuccess;
    dim3 grid(count, st.BH), block(128);
    if (st.es == 2)
        hipLaunchKernelGGL(export_fp_kernel<2>, grid, block, 0, s, st, runs, row_begin, dst_row0, dst_rows, (char *)dst_k, (char *)dst_v);
    else
        hipLaunchKernelGGL(export_fp_kernel<4>, grid, block, 0, s, st, runs, row_begin, dst_row0, dst_rows, (char *)dst_k, (char *)dst_v);
    return hipGetLastError();
}

hipError_t launch_import_fp(const Store &st, const void *src_k, const void *src_v, int nrows, hipStream_t s) {
    if (nrows <= 0) return hipSuccess;
    dim3 grid(nrows, st.BH), block(128);
    if (st.es == 2)
        hipLaunchKernelGGL(import_fp_kernel<2>, grid, block, 0, s, st, (const char *)src_k, (const char *)src_v, nrows);
    else
        hipLaunchKernelGGL(import_fp_kernel<4>, grid, block, 0, s, st, (const char *)src_k, (const char *)src_v, nrows);
    return hipGetLastError();
}

hipError_t launch_compact_fp(const Store &src, const Runs &runs, const Store &dst, int nrows, hipStream_t s) {
    if (nrows <= 0) return hipSuccess;
    dim3 grid(nrows, src.BH), block(128);
    if (src.es == 2)
        hipLaunchKernelGGL(compact_fp_kernel<2>, grid, block, 0, s, src, runs, dst, nrows);
    else
        hipLaunchKernelGGL(compact_fp_kernel<4>, grid, block, 0, s, src, runs, dst, nrows);
    return hipGetLastError();
}

hipError_t launch_export_quant(const Store &st, int which, int nrows, void *dst, hipStream_t s) {
    if (nrows <= 0) return hipSuccess;
    dim3 grid(nrows, st.BH), block(64);
#define EXP(BITS) hipLaunchKernelGGL(export_quant_kernel<BITS>, grid, block, 0, s, st, which, nrows, (char *)dst)
    switch (st.bits) {
        case 4: EXP(4); break;
        case 8: EXP(8); break;
        case 3: EXP(3); break;
        case 5: EXP(5); break;
        case 6: EXP(6); break;
        default: EXP(2); break;
    }
#undef EXP
    return hipGetLastError();
}

hipError_t launch_import_quant(const Store &st, const void *const srcs[6], int nrows, hipStream_t s) {
    if (nrows <= 0) return hipSuccess;
    dim3 grid((nrows + TILE - 1) / TILE, st.BH), block(256);
#define IMP(BITS)                                                                                     \
    hipLaunchKernelGGL(import_quant_kernel<BITS>, grid, block, 0, s, st, (const uint32_t *)srcs[0],   \
                       (const char *)srcs[1], (const char *)srcs[2], (const uint32_t *)srcs[3],       \
                       (const char *)srcs[4], (const char *)srcs[5], nrows)
    switch (st.bits) {
        case 4: IMP(4); break;
        case 8: IMP(8); break;
        case 3: IMP(3); break;
        case 5: IMP(5); break;
        case 6: IMP(6); break;
        default: IMP(2); break;
    }
#undef IMP
    return hipGetLastError();
}

hipError_t launch_affine_quantize(const void *src, int64_t rows, int D, int gs, int bits, int dtype,
                                  uint32_t *wq, void *scales, void *biases, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    const int es = dtype == 2 ? 4 : 2;
#define CALL(DT, BITS)                                                                               \
    hipLaunchKernelGGL((affine_quantize_kernel<DT, BITS>), grid, block, 0, s, (const char *)src, rows, D, gs, \
                       wq, (char *)scales, (char *)biases, es)
    KV_DISPATCH_DT_BITS(dtype, bits, CALL);
#undef CALL
    return hipGetLastError();
}

hipError_t launch_affine_dequantize(const uint32_t *wq, const void *scales, const void *biases,
                                    int64_t rows, int D, int gs, int bits, int dtype, void *dst,
                                    hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    dim3 grid((unsigned)rows), block(128);
#define CALL(DT, BITS)                                                                               \
    hipLaunchKernelGGL((affine_dequantize_kernel<DT, BITS>), grid, block, 0, s, wq, (const char *)scales, \
                       (const char *)biases, rows, D, gs, (char *)dst)
    KV_DISPATCH_DT_BITS(dtype, bits, CALL);
#undef CALL
    return hipGetLastError();
}

// Plain fills and copies of plane memory run as kernels: they see virtual addresses only, so a
// range may span any number of separately mapped physical chunks, and no memset node ends up in
// a stream capture.  16-byte aligned pointers and sizes.
__global__ void __launch_bounds__(256) fill_zero_kernel(u4v *dst, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = u4v{0u, 0u, 0u, 0u};
}
__global__ void __launch_bounds__(256) copy_bytes_kernel(u4v *dst, const u4v *src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// one thread per new page-table entry
__global__ void set_pages_kernel(PageEntry *pt, int first, int count, PageEntry base, size_t sk, size_t sv, size_t sksb, size_t svsb) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    PageEntry e;
    e.k = base.k + (size_t)i * sk;
    e.v = base.v + (size_t)i * sv;
    e.ksb = base.ksb ? base.ksb + (size_t)i * sksb : nullptr;
    e.vsb = base.vsb ? base.vsb + (size_t)i * svsb : nullptr;
    pt[first + i] = e;
}

// grid (pages, 4 planes): the [BH] cells of one plane of one page, 16 bytes per thread and step
__global__ void __launch_bounds__(256) copy_pages_kernel(Store src, Store dst) {
    const PageEntry a = src.pt[blockIdx.x], b = dst.pt[blockIdx.x];
    const int plane = blockIdx.y;
    const char *from = plane == 0 ? a.k : plane == 1 ? a.v : plane == 2 ? a.ksb : a.vsb;
    char *to = plane == 0 ? b.k : plane == 1 ? b.v : plane == 2 ? b.ksb : b.vsb;
    const size_t cell = plane == 0 ? src.k_cell : plane == 1 ? src.v_cell : plane == 2 ? src.ksb_cell : src.vsb_cell;
    const size_t n16 = (size_t)src.BH * cell / 16;
    for (size_t i = threadIdx.x; i < n16; i += 256) reinterpret_cast<u4v *>(to)[i] = reinterpret_cast<const u4v *>(from)[i];
}

hipError_t launch_set_pages(PageEntry *pt, int first, int count, PageEntry base, const size_t stride[4], hipStream_t s) {
    if (count <= 0) return hipSuccess;
    hipLaunchKernelGGL(set_pages_kernel, dim3((count + 63) / 64), dim3(64), 0, s, pt, first, count, base, stride[0], stride[1],
                       stride[2], stride[3]);
    return hipGetLastError();
}

hipError_t launch_copy_pages(const Store &src, const Store &dst, int pages, hipStream_t s) {
    if (pages <= 0) return hipSuccess;
    hipLaunchKernelGGL(copy_pages_kernel, dim3(pages, src.bits ? 4 : 2), dim3(256), 0, s, src, dst);
    return hipGetLastError();
}

hipError_t launch_fill_zero(void *dst, size_t bytes, hipStream_t s) {
    if (bytes == 0) return hipSuccess;
    if (((uintptr_t)dst | bytes) & 15) return hipErrorInvalidValue;
    const size_t n16 = bytes / 16;
    const unsigned grid = (unsigned)std::min<size_t>((n16 + 255) / 256, 256 * 16);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, s, static_cast<u4v *>(dst), n16);
    return hipGetLastError();
}

hipError_t launch_copy_bytes(void *dst, const void *src, size_t bytes, hipStream_t s) {
    if (bytes == 0) return hipSuccess;
    if (((uintptr_t)dst | (uintptr_t)src | bytes) & 15) return hipErrorInvalidValue;
    const size_t n16 = bytes / 16;
    const unsigned grid = (unsigned)std::min<size_t>((n16 + 255) / 256, 256 * 16);
    hipLaunchKernelGGL(copy_bytes_kernel, dim3(grid), dim3(256), 0, s, static_cast<u4v *>(dst), static_cast<const u4v *>(src), n16);
    return hipGetLastError();
}

hipError_t launch_mask_materialize(const kvhip_mask_plan_t &plan, uint8_t *dst, hipStream_t s) {
    if (plan.cols <= 0) return hipSuccess;
    dim3 grid((plan.cols + 255) / 256, plan.rolled ? 1 : (plan.rows < 1024 ? plan.rows : 1024)), block(256);
    hipLaunchKernelGGL(mask_materialize_kernel, grid, block, 0, s, plan, dst);
    return hipGetLastError();
}

}  // namespace kvhip
