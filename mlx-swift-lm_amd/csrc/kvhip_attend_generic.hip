// Generic attention over the page layout: one workgroup per query row, any
// dtype / bit width / head dim / mask.  It is the fallback for shapes the
// matrix-core kernels do not cover and the in-library cross-check for them.
//
// Quantized caches follow the reference's unfused sequence
// (KVCache.swift:2351-2447): q' = T(q*scale), scores = T(q' . K^), mask with
// finfo(T).min fill (or T(scores + mask)), p = T(softmax), out = T(p . V^).
// Full-precision caches follow the fused op (AttentionUtils.swift:86-93):
// float32 inside, excluded keys contribute nothing, one rounding at the output.
#include <algorithm>

#include "kvhip_mask.hpp"

namespace kvhip {

namespace {

constexpr int GT = 256;  // threads per workgroup

__device__ __forceinline__ float block_reduce(float v, bool is_max, float *red) {
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(v, off);
        v = is_max ? fmaxf(v, o) : v + o;
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = red[0];
    for (int w = 1; w < GT / 64; ++w) r = is_max ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

// grid (L, Hq, B)
template <int DT, int BITS>
__global__ void __launch_bounds__(GT)
attend_generic_kernel(AttendArgs a, int slots_pad) {
    extern __shared__ float smem[];  // q' [Dk] | red [4]
    float *qs = smem;
    float *red = smem + a.st.Dk;
    const Store &st = a.st;
    const int l = blockIdx.x, hq = blockIdx.y, b = blockIdx.z;
    const int r = a.Hq / a.Hkv;
    const int bh = b * a.Hkv + hq / r;
    const size_t qrow = ((size_t)(b * a.Hq + hq) * a.L + l);
    float *p = a.workspace + qrow * slots_pad;
    constexpr bool Q = BITS != 0;
    constexpr int BB = Q ? BITS : 4;
    const float fill = finfo_min_dt(DT);

    for (int d = threadIdx.x; d < st.Dk; d += GT) {
        const float qv = Elem<DT>::load(a.q, qrow * st.Dk + d) * a.scale;
        qs[d] = Q ? round_dt<DT>(qv) : qv;
    }
    __syncthreads();

    // ---- scores -------------------------------------------------------------
    float mx = -INFINITY;
    for (int slot = threadIdx.x; slot < slots_pad; slot += GT) {
        const int row = slot < a.slots ? slot_to_row(a.runs, slot) : -1;
        float s = -INFINITY;
        if (row >= 0 && row < a.T) {
            float sum = 0.f;
            if (Q) {
                constexpr int per = 32 / BB;
                const uint32_t *krow = reinterpret_cast<const uint32_t *>(k_row_ptr(st, bh, slot));
                const char *sb = ksb_row_ptr(st, bh, slot);
                for (int g = 0; g < st.Dk / st.gs; ++g) {
                    const float sc = Elem<DT>::load(sb, 2 * g), bi = Elem<DT>::load(sb, 2 * g + 1);
                    if constexpr ((32 % BB) == 0) {
                        for (int w0 = g * st.gs / per; w0 < (g + 1) * st.gs / per; ++w0) {
                            const uint32_t word = krow[w0];
                            for (int i = 0; i < per; ++i) {
                                const uint32_t c = (word >> (i * BB)) & ((1u << BB) - 1u);
                                sum += qs[w0 * per + i] * (sc * (float)c + bi);
                            }
                        }
                    } else {  // 3, 5, 6 bits: codes straddle words of the row's bit stream
                        for (int d = g * st.gs; d < (g + 1) * st.gs; ++d)
                            sum += qs[d] * (sc * (float)stream_code<BB>(krow, d) + bi);
                    }
                }
                s = round_dt<DT>(sum);
            } else {
                const char *kc = k_cell_ptr(st, bh, slot);
                for (int d = 0; d < st.Dk; ++d) sum += qs[d] * Elem<DT>::load(kc + kfp_off(st, slot, d), 0);
                s = sum;
            }
            float add;
            const bool keep = mask_keep(a.mask, b, hq, l, row, a.L, a.T, add);
            if (Q) {
                if (!keep) s = fill;
                else if (a.mask.mode == KVHIP_MASK_ARRAY && a.mask.dtype != KVHIP_BOOL) s = round_dt<DT>(s + add);
            } else {
                s = keep ? s + add : -INFINITY;
            }
        }
        p[slot] = s;
        mx = fmaxf(mx, s);
    }
    mx = block_reduce(mx, true, red);

    // ---- softmax ------------------------------------------------------------
    float den = 0.f;
    for (int slot = threadIdx.x; slot < slots_pad; slot += GT) {
        const float s = p[slot];
        const float e = (s == -INFINITY) ? 0.f : expf(s - mx);
        p[slot] = e;
        den += e;
    }
    den = block_reduce(den, false, red);
    const float inv = den > 0.f ? 1.0f / den : 0.f;
    for (int slot = threadIdx.x; slot < slots_pad; slot += GT) {
        const float w = Q ? round_dt<DT>(__fdiv_rn(p[slot], den > 0.f ? den : 1.f)) : p[slot] * inv;
        p[slot] = w;
    }
    __syncthreads();

    // ---- out = p . V^ ---------------------------------------------------------
    for (int d = threadIdx.x; d < st.Dv; d += GT) {
        float acc = 0.f;
        for (int slot0 = 0; slot0 < slots_pad; slot0 += TILE) {
            const char *vrow = v_cell_ptr(st, bh, slot0) + v_row_off(st, slot0, d);
            const int nt = min(TILE, slots_pad - slot0);
            for (int t = 0; t < nt; ++t) {
                const int slot = slot0 + t;
                const float w = p[slot];
                if (w == 0.f) continue;
                float v;
                if (Q) {
                    const char *sb = vsb_row_ptr(st, bh, slot);
                    const int g = d / st.gs;
                    v = Elem<DT>::load(sb, 2 * g) * (float)v_code_load<BB>(vrow, t) + Elem<DT>::load(sb, 2 * g + 1);
                } else {
                    v = Elem<DT>::load(v_cell_ptr(st, bh, slot) + vfp_off(st, slot, d), 0);
                }
                acc += w * v;
            }
        }
        Elem<DT>::store(a.out, qrow * st.Dv + d, acc);
    }
}

// ---- rows that see no key, after the full-precision tile ran over a dequantized copy of a quantized cache ----
// The reference's quantized sequence fills masked scores with finfo(T).min (KVCache.swift:2441-2445), so a query row
// whose mask excludes every key -- a batch row that is all padding -- weighs all T keys alike: p = T(1 / T), out =
// T(p . V^).  The full-precision tile drops excluded keys and leaves such a row at zero.  This kernel finds those rows
// (boolean arrays: 16 mask bytes per lane and load; index masks: from the bounds) and writes them.
// a.st: the dequantized pages (slots in presented order); grid (row blocks of 64, BH), 256 threads.
template <int DT>
__global__ void __launch_bounds__(GT)
rows_without_keys_kernel(AttendArgs a) {
    __shared__ int empty_s[64];
    __shared__ int any_s;
    const Store &st = a.st;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.y, b = bh / a.Hkv, h = bh % a.Hkv;
    const int r = a.Hq / a.Hkv, R = r * a.L, row0 = blockIdx.x * 64;
    if (tid == 0) any_s = 0;
    __syncthreads();
    for (int i = wave; i < 64; i += GT / 64) {  // one wavefront per query row
        const int rr = row0 + i;
        bool empty = false;
        if (rr < R) {
            const int hq = h * r + rr / a.L, l = rr % a.L;
            if (a.mask.mode == KVHIP_MASK_ARRAY) {
                const uint8_t *mrow = reinterpret_cast<const uint8_t *>(a.mask.data) + (size_t)(b * a.mask.sb + hq * a.mask.sh + l * a.mask.sl);
                bool seen = false;
                for (int base = 0; base < a.T; base += 64 * 16) {  // wave-uniform trips
                    const int j0 = base + lane * 16;
                    if (j0 + 16 <= a.T) {
                        uint32_t w[4];
                        mask_bool_words<4>(a.mask, b, hq, l, j0, w);
                        seen = (w[0] | w[1] | w[2] | w[3]) != 0;
                    } else {
                        for (int j = j0; j < a.T; ++j) seen = seen || mrow[j] != 0;
                    }
                    if (__any(seen)) break;
                }
                empty = !__any(seen);
            } else {
                const SymMask sm = sym_mask_init(a.mask, b, a.L, a.T);
                int lo, hi;
                if (sm.mode == KVHIP_MASK_CAUSAL) {
                    lo = 0;
                    hi = a.T - a.L + l;
                } else {
                    lo = sm.pad_b;
                    hi = min(sm.offset + l, sm.len_b - 1);
                    if (sm.window > 0) lo = max(lo, sm.offset + l - sm.window + 1);
                }
                empty = max(lo, 0) > min(hi, a.T - 1);
            }
        }
        if (lane == 0) {
            empty_s[i] = empty;
            if (empty) any_s = 1;
        }
    }
    __syncthreads();
    if (!any_s) return;
    const float p = round_dt<DT>(1.0f / (float)a.T);
    constexpr int EPC = DT == 2 ? 4 : 8;  // tokens per 16-byte chunk of a V tile
    for (int d = tid; d < st.Dv; d += GT) {
        float sum = 0.f;
        for (int slot0 = 0; slot0 < a.T; slot0 += EPC) {
            const uint4 w = *reinterpret_cast<const uint4 *>(v_cell_ptr(st, bh, slot0) + vfp_off(st, slot0, d));  // EPC tokens of column d
            const int n = min(EPC, a.T - slot0);
            for (int e = 0; e < n; ++e) sum += Elem<DT>::load(&w, e);
        }
        const float v = p * sum;
        for (int i = 0; i < 64; ++i) {
            if (!empty_s[i]) continue;
            const int rr = row0 + i, hq = h * r + rr / a.L, l = rr % a.L;
            Elem<DT>::store(a.out, ((size_t)(b * a.Hq + hq) * a.L + l) * st.Dv + d, v);
        }
    }
}

}  // namespace

bool mask_may_leave_rows_without_keys(const AttendArgs &a) {
    const MaskDev &m = a.mask;
    if (m.mode == KVHIP_MASK_NONE) return false;
    if (m.mode == KVHIP_MASK_CAUSAL) return a.T < a.L;
    if (m.mode == KVHIP_MASK_ARRAY) return m.dtype == KVHIP_BOOL;
    if (m.lengths || m.left_pad) return true;  // per-batch bounds in device memory
    for (int e = 0; e < 2; ++e) {  // the kept range [max(0, offset + l - window + 1), min(offset + l, T - 1)] is narrowest at an end
        const int l = e ? a.L - 1 : 0;
        const int lo = m.window > 0 ? std::max(0, m.offset + l - m.window + 1) : 0, hi = std::min(m.offset + l, a.T - 1);
        if (lo > hi) return true;
    }
    return false;
}

hipError_t launch_rows_without_keys(const AttendArgs &a, hipStream_t s) {
    const dim3 grid(((a.Hq / a.Hkv) * a.L + 63) / 64, a.st.BH), block(GT);
    if (a.st.dtype == KVHIP_F16) hipLaunchKernelGGL(rows_without_keys_kernel<0>, grid, block, 0, s, a);
    else if (a.st.dtype == KVHIP_BF16) hipLaunchKernelGGL(rows_without_keys_kernel<1>, grid, block, 0, s, a);
    else hipLaunchKernelGGL(rows_without_keys_kernel<2>, grid, block, 0, s, a);
    return hipGetLastError();
}

static int pad32(int n) { return (n + 31) & ~31; }

size_t attend_generic_workspace(const AttendArgs &a) {
    return (size_t)a.B * a.Hq * a.L * pad32(a.slots) * sizeof(float);
}

hipError_t launch_attend_generic(const AttendArgs &a, hipStream_t s) {
    dim3 grid(a.L, a.Hq, a.B), block(GT);
    const size_t lds = (a.st.Dk + 8) * sizeof(float);
    const int sp = pad32(a.slots);
#define GEN(DT, BITS) hipLaunchKernelGGL((attend_generic_kernel<DT, BITS>), grid, block, lds, s, a, sp)
#define GEN_DT(BITS)                                        \
    do {                                                    \
        if (a.st.dtype == 0) GEN(0, BITS);                  \
        else if (a.st.dtype == 1) GEN(1, BITS);             \
        else GEN(2, BITS);                                  \
    } while (0)
    switch (a.st.bits) {
        case 0: GEN_DT(0); break;
        case 2: GEN_DT(2); break;
        case 4: GEN_DT(4); break;
        case 3: GEN_DT(3); break;
        case 5: GEN_DT(5); break;
        case 6: GEN_DT(6); break;
        default: GEN_DT(8); break;
    }
#undef GEN_DT
#undef GEN
    return hipGetLastError();
}

}  // namespace kvhip
