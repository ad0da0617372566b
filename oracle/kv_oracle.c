/*
 * kv_oracle.c -- scalar C restatement of the reference's CPU path for the
 * KV-cache hot path.  TEST INFRASTRUCTURE ONLY: it is loaded by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py, never by
 * the product library.
 *
 * It restates the op sequence the reference issues for one quantized decode
 * step (Libraries/MLXLMCommon/KVCache.swift):
 *   kvo_affine_quantize   MLX.quantized         :1069-1070 (also :506,:508,:975)
 *   kvo_affine_dequantize MLX.dequantized       :1197,:1200
 *   kvo_qsdpa             quantizedScaledDotProductAttention :2351-2447
 *                         (queries*scale, quantizedMM(transpose:true), mask,
 *                          softmax, quantizedMM(transpose:false); the scores
 *                          array is materialised, as in the reference)
 *   kvo_sdpa              MLXFast.scaledDotProductAttention via
 *                         AttentionUtils.swift:86-93
 *
 * The arithmetic of these ops belongs to the third-party dependency
 * ml-explore/mlx-swift (0.31.6 ..< 0.32.0, Package.swift:64), which is not
 * part of the reference checkout; its published CPU algorithm is restated
 * here.  kvo_affine_quantize is pinned against that published loop by the
 * hand-worked known answers of tests/quantizer_kats.py (and by closed forms,
 * invariants and the independent numpy restatement in kv_oracle.py); against
 * an output of MLX itself, which the reference does not hold, code / scale /
 * bias bits stay "parity unpinned", and so does the accumulation order and
 * dtype inside quantizedMM / softmax (softmax(precise: false) accumulates in T
 * on MLX's CPU backend, in float32 here).
 *
 * Arrays are float32 holding values representable in the logical dtype T
 * (0 = float16, 1 = bfloat16, 2 = float32); kvo_round applies T's rounding
 * wherever the reference materialises an array.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* float32 -> float16 bits, round to nearest even */
static inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x = f2u(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) return (uint16_t)(sign | (ax > 0x7f800000u ? 0x7e00u : 0x7c00u));
    if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x38800000u) { /* subnormal or zero in f16 */
        if (ax < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
        int e = (int)(ax >> 23);
        uint32_t m = (ax & 0x7fffffu) | 0x800000u;
        int shift = 126 - e; /* m * 2^(e-150) expressed in units of 2^-24 */
        uint32_t r = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (r & 1u))) r++;
        return (uint16_t)(sign | r);
    }
    uint32_t r = ax - 0x38000000u; /* rebias exponent */
    uint32_t rem = r & 0x1fffu;
    r >>= 13;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
    return (uint16_t)(sign | r);
}

static inline float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    if (e == 0) {
        if (m == 0) return u2f(sign);
        float v = (float)m * 5.9604644775390625e-08f; /* 2^-24 */
        return sign ? -v : v;
    }
    if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
    return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

static inline uint16_t f32_to_bf16_bits(float f) {
    uint32_t x = f2u(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
    uint32_t r = ((x >> 16) & 1u) + 0x7fffu;
    return (uint16_t)((x + r) >> 16);
}

float kvo_round(float x, int dtype) {
    if (dtype == 0) return f16_bits_to_f32(f32_to_f16_bits(x));
    if (dtype == 1) return u2f((uint32_t)f32_to_bf16_bits(x) << 16);
    return x;
}

static inline float finfo_min(int dtype) {
    if (dtype == 0) return -65504.0f;
    if (dtype == 1) return -3.3895313892515355e38f;
    return -3.4028234663852886e38f;
}

/* MLX.quantized, affine mode.  w: [rows, D]; wq: [rows, D*bits/32];
 * scales/biases: [rows, D/gs] (float32 holding T values). */
void kvo_affine_quantize(const float *w, int64_t rows, int D, int gs, int bits, int dtype,
                         uint32_t *wq, float *scales, float *biases) {
    const float n_bins = (float)((1 << bits) - 1);
    const float eps = 1e-7f;
    const int G = D / gs;
    const int per = 32 / bits;
    const int W = D / per;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float *row = w + r * D;
        uint32_t *out = wq + r * W;
        for (int i = 0; i < W; ++i) out[i] = 0;
        for (int g = 0; g < G; ++g) {
            const float *x = row + g * gs;
            float w_min = INFINITY, w_max = -INFINITY;
            for (int j = 0; j < gs; ++j) {
                w_max = fmaxf(w_max, x[j]);
                w_min = fminf(w_min, x[j]);
            }
            int mask = fabsf(w_min) > fabsf(w_max);
            float scale = fmaxf((w_max - w_min) / n_bins, eps);
            scale = mask ? scale : -scale;
            float edge = mask ? w_min : w_max;
            float q0 = rintf(edge / scale);
            float bias = 0.0f;
            if (q0 != 0.0f) {
                scale = edge / q0;
                bias = edge;
            }
            for (int j = 0; j < gs; ++j) {
                float q = rintf((x[j] - bias) / scale);
                q = fminf(fmaxf(q, 0.0f), n_bins);
                int d = g * gs + j;
                out[d / per] |= ((uint32_t)q) << ((d % per) * bits);
            }
            scales[r * G + g] = kvo_round(scale, dtype);
            biases[r * G + g] = kvo_round(bias, dtype);
        }
    }
}

static inline float deq_elem(const uint32_t *wq, const float *s, const float *b, int d, int gs,
                             int bits) {
    const int per = 32 / bits;
    uint32_t c = (wq[d / per] >> ((d % per) * bits)) & ((1u << bits) - 1u);
    return s[d / gs] * (float)c + b[d / gs];
}

/* MLX.dequantized: out[rows, D] = T(scale*code + bias) */
void kvo_affine_dequantize(const uint32_t *wq, const float *scales, const float *biases,
                           int64_t rows, int D, int gs, int bits, int dtype, float *out) {
    const int G = D / gs, W = D * bits / 32;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int d = 0; d < D; ++d)
            out[r * D + d] = kvo_round(deq_elem(wq + r * W, scales + r * G, biases + r * G, d, gs, bits), dtype);
}

/*
 * Mask descriptor shared by kvo_qsdpa / kvo_sdpa.
 *   mode 0: none   1: causal (query i sees keys j <= T-L+i)
 *   mode 2: bool array   3: additive float array
 * Array masks are addressed as mask[b*sb + h*sh + l*sl + t] with h the QUERY
 * head; a stride of 0 broadcasts that axis.
 */
typedef struct {
    int32_t mode;
    const uint8_t *bool_data;
    const float *add_data;
    int64_t sb, sh, sl;
} kvo_mask;

/*
 * quantizedScaledDotProductAttention, unfused as in the reference:
 *   q' = T(q*scale); scores = T(q' . K^); mask; p = T(softmax(scores)); out = T(p . V^)
 * q: [B,Hq,L,Dk]; K codes [B,Hkv,T,Dk*bits/32] + scales/biases [B,Hkv,T,Dk/gs];
 * V likewise with Dv; out: [B,Hq,L,Dv].  `scores_scratch` holds B*Hq*L*T floats.
 */
void kvo_qsdpa(const float *q, const uint32_t *kw, const float *ks, const float *kb,
               const uint32_t *vw, const float *vs, const float *vb, int B, int Hq, int Hkv, int L,
               int T, int Dk, int Dv, int gs, int bits, int dtype, float scale,
               const kvo_mask *mask, float *scores_scratch, float *out) {
    const int r = Hq / Hkv;
    const int Wk = Dk * bits / 32, Wv = Dv * bits / 32, Gk = Dk / gs, Gv = Dv / gs;
    const float fill = finfo_min(dtype);
    const int per = 32 / bits;
    const uint32_t cmask = (1u << bits) - 1u;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int b = 0; b < B; ++b) {
        for (int hq = 0; hq < Hq; ++hq) {
            const int hk = hq / r;
            const int64_t kvrow0 = ((int64_t)b * Hkv + hk) * T;
            float *qs = (float *)malloc(sizeof(float) * Dk);
            float *acc = (float *)malloc(sizeof(float) * Dv);
            for (int l = 0; l < L; ++l) {
                const float *qrow = q + (((int64_t)b * Hq + hq) * L + l) * Dk;
                float *srow = scores_scratch + (((int64_t)b * Hq + hq) * L + l) * T;
                for (int d = 0; d < Dk; ++d) qs[d] = kvo_round(qrow[d] * scale, dtype);
                /* scores = quantizedMM(q', K, transpose: true) */
                for (int t = 0; t < T; ++t) {
                    const uint32_t *w = kw + (kvrow0 + t) * Wk;
                    const float *s = ks + (kvrow0 + t) * Gk;
                    const float *bb = kb + (kvrow0 + t) * Gk;
                    float sum = 0.0f;
                    for (int g = 0; g < Gk; ++g) {
                        float sc = s[g], bi = bb[g];
                        for (int j = 0; j < gs; ++j) {
                            int d = g * gs + j;
                            uint32_t c = (w[d / per] >> ((d % per) * bits)) & cmask;
                            sum += qs[d] * (sc * (float)c + bi);
                        }
                    }
                    float sv = kvo_round(sum, dtype);
                    if (mask) {
                        if (mask->mode == 1) {
                            if (!(l + (T - L) >= t)) sv = fill;
                        } else if (mask->mode == 2) {
                            if (!mask->bool_data[b * mask->sb + hq * mask->sh + l * mask->sl + t]) sv = fill;
                        } else if (mask->mode == 3) {
                            sv = kvo_round(sv + mask->add_data[b * mask->sb + hq * mask->sh + l * mask->sl + t], dtype);
                        }
                    }
                    srow[t] = sv;
                }
                /* softmax(axis: -1) */
                float mx = -INFINITY;
                for (int t = 0; t < T; ++t) mx = fmaxf(mx, srow[t]);
                float den = 0.0f;
                for (int t = 0; t < T; ++t) {
                    srow[t] = expf(srow[t] - mx);
                    den += srow[t];
                }
                for (int t = 0; t < T; ++t) srow[t] = kvo_round(srow[t] / den, dtype);
                /* out = quantizedMM(p, V, transpose: false) */
                for (int d = 0; d < Dv; ++d) acc[d] = 0.0f;
                for (int t = 0; t < T; ++t) {
                    const float p = srow[t];
                    if (p == 0.0f) continue;
                    const uint32_t *w = vw + (kvrow0 + t) * Wv;
                    const float *s = vs + (kvrow0 + t) * Gv;
                    const float *bb = vb + (kvrow0 + t) * Gv;
                    for (int g = 0; g < Gv; ++g) {
                        float sc = s[g], bi = bb[g];
                        for (int j = 0; j < gs; ++j) {
                            int d = g * gs + j;
                            uint32_t c = (w[d / per] >> ((d % per) * bits)) & cmask;
                            acc[d] += p * (sc * (float)c + bi);
                        }
                    }
                }
                float *orow = out + (((int64_t)b * Hq + hq) * L + l) * Dv;
                for (int d = 0; d < Dv; ++d) orow[d] = kvo_round(acc[d], dtype);
            }
            free(qs);
            free(acc);
        }
    }
}

/* MLXFast.scaledDotProductAttention: float32 inside, one rounding at the output.
 * k: [B,Hkv,T,Dk], v: [B,Hkv,T,Dv]. Bool masks exclude (-inf), float masks add. */
void kvo_sdpa(const float *q, const float *k, const float *v, int B, int Hq, int Hkv, int L, int T,
              int Dk, int Dv, int dtype, float scale, const kvo_mask *mask, float *out) {
    const int r = Hq / Hkv;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (int b = 0; b < B; ++b) {
        for (int hq = 0; hq < Hq; ++hq) {
            const int hk = hq / r;
            float *srow = (float *)malloc(sizeof(float) * T);
            float *acc = (float *)malloc(sizeof(float) * Dv);
            for (int l = 0; l < L; ++l) {
                const float *qrow = q + (((int64_t)b * Hq + hq) * L + l) * Dk;
                float mx = -INFINITY;
                for (int t = 0; t < T; ++t) {
                    const float *krow = k + (((int64_t)b * Hkv + hk) * T + t) * Dk;
                    float sum = 0.0f;
                    for (int d = 0; d < Dk; ++d) sum += (qrow[d] * scale) * krow[d];
                    if (mask) {
                        if (mask->mode == 1) {
                            if (!(l + (T - L) >= t)) sum = -INFINITY;
                        } else if (mask->mode == 2) {
                            if (!mask->bool_data[b * mask->sb + hq * mask->sh + l * mask->sl + t]) sum = -INFINITY;
                        } else if (mask->mode == 3) {
                            sum += mask->add_data[b * mask->sb + hq * mask->sh + l * mask->sl + t];
                        }
                    }
                    srow[t] = sum;
                    mx = fmaxf(mx, sum);
                }
                float den = 0.0f;
                for (int t = 0; t < T; ++t) {
                    srow[t] = expf(srow[t] - mx);
                    den += srow[t];
                }
                for (int d = 0; d < Dv; ++d) acc[d] = 0.0f;
                for (int t = 0; t < T; ++t) {
                    const float p = srow[t] / den;
                    const float *vrow = v + (((int64_t)b * Hkv + hk) * T + t) * Dv;
                    for (int d = 0; d < Dv; ++d) acc[d] += p * vrow[d];
                }
                float *orow = out + (((int64_t)b * Hq + hq) * L + l) * Dv;
                for (int d = 0; d < Dv; ++d) orow[d] = kvo_round(acc[d], dtype);
            }
            free(srow);
            free(acc);
        }
    }
}

int kvo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
