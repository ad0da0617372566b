// Device-side element conversion and the affine quantizer core shared by the
// append, import/export and standalone quantize kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "kvhip_internal.hpp"

namespace kvhip {

// DT: 0 float16, 1 bfloat16, 2 float32 (kvhip_dtype)
template <int DT> struct Elem;
template <> struct Elem<0> {
    using type = uint16_t;
    static __device__ __forceinline__ float load(const void *p, size_t i) {
        return __half2float(reinterpret_cast<const __half *>(p)[i]);
    }
    static __device__ __forceinline__ void store(void *p, size_t i, float v) {
        reinterpret_cast<__half *>(p)[i] = __float2half_rn(v);
    }
};
template <> struct Elem<1> {
    using type = uint16_t;
    static __device__ __forceinline__ float load(const void *p, size_t i) {
        return __uint_as_float((uint32_t) reinterpret_cast<const uint16_t *>(p)[i] << 16);
    }
    static __device__ __forceinline__ uint16_t bits(float v) {
        uint32_t x = __float_as_uint(v);
        if ((x & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
        return (uint16_t)((x + (((x >> 16) & 1u) + 0x7fffu)) >> 16);
    }
    static __device__ __forceinline__ void store(void *p, size_t i, float v) {
        reinterpret_cast<uint16_t *>(p)[i] = bits(v);
    }
};
template <> struct Elem<2> {
    using type = float;
    static __device__ __forceinline__ float load(const void *p, size_t i) {
        return reinterpret_cast<const float *>(p)[i];
    }
    static __device__ __forceinline__ void store(void *p, size_t i, float v) {
        reinterpret_cast<float *>(p)[i] = v;
    }
};

// Round a float to dtype DT and back (the value an array of that dtype holds).
template <int DT> __device__ __forceinline__ float round_dt(float v) {
    if (DT == 0) return __half2float(__float2half_rn(v));
    if (DT == 1) return __uint_as_float((uint32_t)Elem<1>::bits(v) << 16);
    return v;
}

__device__ __forceinline__ float finfo_min_dt(int dt) {
    return dt == 0 ? -65504.0f : (dt == 1 ? -3.3895313892515355e38f : -3.4028234663852886e38f);
}

// Two floats -> two 16-bit floats in one dword (low half first), rounded to nearest even by the
// packed converts of gfx950 (v_cvt_pk_f16_f32 / v_cvt_pk_bf16_f32): one instruction per pair.
typedef float kv_f2 __attribute__((ext_vector_type(2)));
typedef _Float16 kv_h2 __attribute__((ext_vector_type(2)));
typedef __bf16 kv_b2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_h2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((kv_f2{lo, hi}), kv_h2));
}
__device__ __forceinline__ uint32_t pk_bf2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((kv_f2{lo, hi}), kv_b2));
}

// Affine parameters of one group from its extrema, in float32, step for step as
// MLX's CPU quantizer computes them (call sites KVCache.swift:1069-1070).
__device__ __forceinline__ void affine_params(float w_min, float w_max, float n_bins, float &scale,
                                              float &bias) {
    const float eps = 1e-7f;
    const bool mask = fabsf(w_min) > fabsf(w_max);
    float s = fmaxf(__fdiv_rn(__fsub_rn(w_max, w_min), n_bins), eps);
    s = mask ? s : -s;
    const float edge = mask ? w_min : w_max;
    const float q0 = rintf(__fdiv_rn(edge, s));
    bias = 0.0f;
    if (q0 != 0.0f) {
        s = __fdiv_rn(edge, q0);
        bias = edge;
    }
    scale = s;
}

__device__ __forceinline__ uint32_t affine_code(float w, float scale, float bias, float n_bins) {
    float q = rintf(__fdiv_rn(__fsub_rn(w, bias), scale));
    q = fminf(fmaxf(q, 0.0f), n_bins);
    return (uint32_t)q;
}

// Min/max over GL (4, 8 or 16) adjacent lanes without LDS round trips: two quad permutes, then
// the mirror of each half row and of each row (the lanes of a quad, then of a half row, already
// agree, so the mirrored lane holds the other half's result).  Minimum and maximum do not depend
// on the order of the reduction.
// Each step is one instruction per value, the permute being an operand modifier (through the
// permuting-move builtin a step came out as a copy, the move, a quieting maximum and the minimum:
// 24 instructions per reduction of two values at GL = 8 instead of 6).  A register written by a
// vector instruction may be read through a permute two wait states later at the earliest: the
// other value's instruction and one s_nop stand between; the leading s_nop covers whatever wrote
// the inputs (and a write of the execution mask, five wait states).
#define KV_MINMAX_STEP(CTRL)                                                \
    "v_min_f32_dpp %0, %0, %0 " CTRL " row_mask:0xf bank_mask:0xf\n\t"      \
    "v_max_f32_dpp %1, %1, %1 " CTRL " row_mask:0xf bank_mask:0xf\n\t"      \
    "s_nop 0\n\t"
template <int GL> __device__ __forceinline__ void group_minmax_dpp(float &mn, float &mx) {
    static_assert(GL == 4 || GL == 8 || GL == 16, "lanes per quantization group");
    if constexpr (GL == 4)
        asm volatile("s_nop 4\n\t" KV_MINMAX_STEP("quad_perm:[1,0,3,2]") KV_MINMAX_STEP("quad_perm:[2,3,0,1]") : "+v"(mn), "+v"(mx));
    else if constexpr (GL == 8)
        asm volatile("s_nop 4\n\t" KV_MINMAX_STEP("quad_perm:[1,0,3,2]") KV_MINMAX_STEP("quad_perm:[2,3,0,1]")
                     KV_MINMAX_STEP("row_half_mirror") : "+v"(mn), "+v"(mx));
    else
        asm volatile("s_nop 4\n\t" KV_MINMAX_STEP("quad_perm:[1,0,3,2]") KV_MINMAX_STEP("quad_perm:[2,3,0,1]")
                     KV_MINMAX_STEP("row_half_mirror") KV_MINMAX_STEP("row_mirror") : "+v"(mn), "+v"(mx));
}
#undef KV_MINMAX_STEP

// Min/max over a group of `width` (32 or 64) adjacent lanes of a wavefront; every lane gets its group's values.
// Rows of 16 lanes are reduced with the permutes above; the four rows' results are then read into scalar registers
// and combined there (twelve LDS permutes with their latencies, which is what the reduction cost as a butterfly of
// __shfl_xor, held a single-row append up for a microsecond per 64 elements).  Minimum and maximum do not depend on
// the order of the reduction.
__device__ __forceinline__ void group_minmax(float &mn, float &mx, int width) {
    group_minmax_dpp<16>(mn, mx);
    const int mi = __builtin_bit_cast(int, mn), xi = __builtin_bit_cast(int, mx);
    const float n0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(mi, 0)), n1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(mi, 16));
    const float n2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(mi, 32)), n3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(mi, 48));
    const float x0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 0)), x1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 16));
    const float x2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 32)), x3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 48));
    const float nlo = fminf(n0, n1), nhi = fminf(n2, n3), xlo = fmaxf(x0, x1), xhi = fmaxf(x2, x3);
    if (width >= 64) {
        mn = fminf(nlo, nhi);
        mx = fmaxf(xlo, xhi);
    } else {  // 32: lanes 0..31 and 32..63 are two groups
        const bool upper = (threadIdx.x & 32) != 0;
        mn = upper ? nhi : nlo;
        mx = upper ? xhi : xlo;
    }
}

// OR-combine `v` across `width` (2, 4, 8 or 16) adjacent lanes: one instruction per step, the permute an operand modifier.
__device__ __forceinline__ uint32_t group_or(uint32_t v, int width) {
#define KV_OR_STEP(CTRL) "v_or_b32_dpp %0, %0, %0 " CTRL " row_mask:0xf bank_mask:0xf\n\ts_nop 1\n\t"
    if (width >= 2) asm volatile("s_nop 4\n\t" KV_OR_STEP("quad_perm:[1,0,3,2]") : "+v"(v));
    if (width >= 4) asm volatile(KV_OR_STEP("quad_perm:[2,3,0,1]") : "+v"(v));
    if (width >= 8) asm volatile(KV_OR_STEP("row_half_mirror") : "+v"(v));
    if (width >= 16) asm volatile(KV_OR_STEP("row_mirror") : "+v"(v));
#undef KV_OR_STEP
    return v;
}

// One wavefront quantizes one row of D elements (groupwise affine, MLX's CPU algorithm).
// `load(d)` hands element d of the row as float; `code_sink(d, code)` receives every code.
// Optional outputs:
//   k_words   packed codes in MLX order (D*BITS/32 words)
//   sb_row    (scale, bias) pairs of dtype DT per group
//   scales / biases   separate arrays of dtype DT per group
template <int DT, int BITS, class LOAD, class SINK>
__device__ __forceinline__ void quantize_row_wave_from(LOAD load, int D, int gs, int lane,
                                                       uint32_t *k_words, SINK code_sink, void *sb_row,
                                                       void *scales, void *biases) {
    const float nb = (float)((1 << BITS) - 1);
    const int K = gs > 64 ? gs / 64 : 1;
    const int width = gs < 64 ? gs : 64;
    constexpr int per = 32 / BITS;
    for (int base = 0; base < D; base += 64 * K) {
        float w[2] = {0.f, 0.f};
        float mn = INFINITY, mx = -INFINITY;
        for (int k = 0; k < K; ++k) {
            const int d = base + k * 64 + lane;
            if (d < D) {
                w[k] = load(d);
                mn = fminf(mn, w[k]);
                mx = fmaxf(mx, w[k]);
            }
        }
        group_minmax(mn, mx, width);
        float scale, bias;
        affine_params(mn, mx, nb, scale, bias);
        for (int k = 0; k < K; ++k) {
            const int d = base + k * 64 + lane;
            const bool valid = d < D;
            const uint32_t code = valid ? affine_code(w[k], scale, bias, nb) : 0u;
            if (k_words) {
                if constexpr ((32 % BITS) == 0) {
                    const uint32_t word = group_or(code << ((d % per) * BITS), per);
                    if (valid && (lane % per) == 0) k_words[d / per] = word;
                } else {
                    // 3, 5 and 6 bits: the 64 codes of this pass are 2 BITS whole words of the row's bit stream;
                    // lane w < 2 BITS collects the codes that touch word w (at most 32 / BITS + 2 of them)
                    const int j0 = (32 * lane) / BITS;
                    uint32_t word = 0u;
#pragma unroll
                    for (int i = 0; i < 32 / BITS + 2; ++i) {
                        const int j = j0 + i;
                        const uint32_t c = __shfl(code, j & 63);
                        if (j < 64 && j * BITS < 32 * lane + 32) word |= stream_bits(c, j * BITS, lane);
                    }
                    const int wi = (base + k * 64) * BITS / 32 + lane;
                    if (lane < 2 * BITS && wi < D * BITS / 32) k_words[wi] = word;
                }
            }
            if (valid) code_sink(d, code);
        }
        const int d0 = base + lane;
        if (d0 < D && (d0 % gs) == 0) {
            const int g = d0 / gs;
            if (sb_row) {
                Elem<DT>::store(sb_row, 2 * g, scale);
                Elem<DT>::store(sb_row, 2 * g + 1, bias);
            }
            if (scales) {
                Elem<DT>::store(scales, g, scale);
                Elem<DT>::store(biases, g, bias);
            }
        }
    }
}

typedef uint32_t kv_u4 __attribute__((ext_vector_type(4)));
// code j of a unit whose words hold a little-endian bit stream (j and BITS constant once unrolled)
template <int BITS, int N> __device__ __forceinline__ uint32_t stream_code_at(const uint32_t (&w)[N], int j) {
    const int bit = j * BITS, wi = bit >> 5, sh = bit & 31;
    uint32_t v = w[wi] >> sh;
    if (sh + BITS > 32) v |= w[wi + 1 < N ? wi + 1 : wi] << ((32 - sh) & 31);
    return v & ((1u << BITS) - 1u);
}
// codes 8 c .. 8 c + 7 of such a unit as four float16 pairs with `mag` OR-ed over them: 0x64006400 (in a vector
// register) gives (1024 + code, 1024 + code), 0 leaves the codes as the subnormals code * 2^-24.  A pair of adjacent codes is cut out as one field of 2 BITS bits; for 2, 3 and 5 bits the field
// times (1 + 2^(16 - BITS)) has the first code at bit 0 and the second at bit 16 (what else the product holds lies
// between them and cannot carry into bit 16: the low part stays below 2^16), so one 24-bit multiply and one
// mask-and-OR finish the pair.  Six-bit codes would carry (63 + 63 * 64 + 63 * 1024 > 2^16) and are placed one by one.
template <int BITS, int N> __device__ __forceinline__ kv_u4 stream_chunk(const uint32_t (&w)[N], int c, uint32_t mag) {
    kv_u4 o;
    constexpr uint32_t M1 = (1u << BITS) - 1u;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (BITS == 6) {
            o[i] = stream_code_at<BITS, N>(w, 8 * c + 2 * i) | (stream_code_at<BITS, N>(w, 8 * c + 2 * i + 1) << 16) | mag;
        } else {
            const int bit = (8 * c + 2 * i) * BITS, wi = bit >> 5, sh = bit & 31;
            uint32_t x = w[wi] >> sh;
            if (sh + 2 * BITS > 32) x = __builtin_amdgcn_alignbit(w[wi + 1 < N ? wi + 1 : wi], w[wi], sh);
            x &= (1u << (2 * BITS)) - 1u;
            const uint32_t y = __umul24(x, 1u + (1u << (16 - BITS)));
            o[i] = (y & (M1 | (M1 << 16))) | mag;
        }
    }
    return o;
}

}  // namespace kvhip
