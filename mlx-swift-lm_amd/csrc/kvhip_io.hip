// Append (full precision and quantize-on-append), import/export between the
// page layout and the reference's dense array layout, ring-order gather, and
// the standalone affine quantizer.
#include "kvhip_device.hpp"

namespace kvhip {

namespace {

template <int BITS> __device__ __forceinline__ uint32_t read_v_code(const char *cell, int unit, int e) {
    if (BITS == 4) return (reinterpret_cast<const uint32_t *>(cell)[unit] >> (4 * e)) & 15u;
    if (BITS == 8) return reinterpret_cast<const uint8_t *>(cell)[(size_t)unit * 8 + e];
    return (reinterpret_cast<const uint16_t *>(cell)[unit] >> (2 * e)) & 3u;
}

// One wavefront quantizes one row of D elements.  Optional outputs:
//   k_words   packed codes in MLX order (D*BITS/32 words)
//   code_out  one byte per element (for the transposed V assembly)
//   sb_row    (scale,bias) pairs of dtype DT per group
//   scales/biases separate arrays of dtype DT per group
template <int DT, int BITS>
__device__ __forceinline__ void quantize_row_wave(const void *src, int D, int gs, int lane,
                                                  uint32_t *k_words, uint8_t *code_out, void *sb_row,
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
                w[k] = Elem<DT>::load(src, d);
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
                const uint32_t word = group_or(code << ((d % per) * BITS), per);
                if (valid && (lane % per) == 0) k_words[d / per] = word;
            }
            if (code_out && valid) code_out[d] = (uint8_t)code;
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

// grid (rows, BH): K rows copied in natural order, V elements scattered into octets.
template <int ES>
__global__ void append_fp_kernel(Store st, const char *keys, const char *values, int L, int src0,
                                 int slot0) {
    const int bh = blockIdx.y;
    const int i = blockIdx.x;
    const int slot = slot0 + i;
    const int l = src0 + i;
    using E = typename std::conditional<ES == 2, uint16_t, uint32_t>::type;
    const E *ks = reinterpret_cast<const E *>(keys) + ((size_t)bh * L + l) * st.Dk;
    E *kd = reinterpret_cast<E *>(const_cast<char *>(k_row_ptr(st, bh, slot)));
    for (int d = threadIdx.x; d < st.Dk; d += blockDim.x) kd[d] = ks[d];
    const E *vs = reinterpret_cast<const E *>(values) + ((size_t)bh * L + l) * st.Dv;
    E *vd = reinterpret_cast<E *>(const_cast<char *>(v_cell_ptr(st, bh, slot)));
    const int ub = v_unit_base(slot, st.Dv);
    const int e = v_pos(slot);
    for (int d = threadIdx.x; d < st.Dv; d += blockDim.x) vd[(size_t)(ub + d) * 8 + e] = vs[d];
}

// grid (32-token blocks touched, BH), 256 threads.  Each wavefront quantizes rows
// of the block; V codes are staged as bytes in LDS and then merged into the
// octet words, touching only the positions this append writes.
template <int DT, int BITS>
__global__ void __launch_bounds__(256)
append_quant_kernel(Store st, const char *keys, const char *values, int L, int src0, int slot0, int n) {
    extern __shared__ uint8_t vcodes[];  // [32][Dv]
    const int bh = blockIdx.y;
    const int blk = (slot0 >> 5) + blockIdx.x;
    const int lo = max(slot0, blk * 32);
    const int hi = min(slot0 + n, blk * 32 + 32);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    for (int slot = lo + wave; slot < hi; slot += 4) {
        const int l = src0 + (slot - slot0);
        const char *krow = keys + ((size_t)bh * L + l) * st.Dk * st.es;
        const char *vrow = values + ((size_t)bh * L + l) * st.Dv * st.es;
        quantize_row_wave<DT, BITS>(krow, st.Dk, st.gs, lane,
                                    reinterpret_cast<uint32_t *>(const_cast<char *>(k_row_ptr(st, bh, slot))),
                                    nullptr, const_cast<char *>(ksb_row_ptr(st, bh, slot)), nullptr, nullptr);
        quantize_row_wave<DT, BITS>(vrow, st.Dv, st.gs, lane, nullptr, vcodes + (slot & 31) * st.Dv,
                                    const_cast<char *>(vsb_row_ptr(st, bh, slot)), nullptr, nullptr);
    }
    __syncthreads();
    char *cell = const_cast<char *>(v_cell_ptr(st, bh, blk * 32));
    const int blk_in_page = ((blk * 32) & (PAGE - 1)) >> 5;
    const int units = 4 * st.Dv;
    for (int u = threadIdx.x; u < units; u += blockDim.x) {
        const int j = u / st.Dv, d = u - j * st.Dv;
        uint64_t nbits = 0, mbits = 0;
        for (int e = 0; e < 8; ++e) {
            const int tl = 4 * j + (e & 3) + 16 * (e >> 2);
            const int slot = blk * 32 + tl;
            if (slot >= lo && slot < hi) {
                nbits |= (uint64_t)vcodes[tl * st.Dv + d] << (e * BITS);
                mbits |= (uint64_t)((1u << BITS) - 1u) << (e * BITS);
            }
        }
        if (mbits == 0) continue;
        const int unit = (blk_in_page * 4 + j) * st.Dv + d;
        if (BITS == 4) {
            uint32_t *p = reinterpret_cast<uint32_t *>(cell) + unit;
            const uint32_t m = (uint32_t)mbits;
            *p = (m == 0xffffffffu) ? (uint32_t)nbits : ((*p & ~m) | (uint32_t)nbits);
        } else if (BITS == 8) {
            uint64_t *p = reinterpret_cast<uint64_t *>(cell) + unit;
            *p = (mbits == ~0ull) ? nbits : ((*p & ~mbits) | nbits);
        } else {
            uint16_t *p = reinterpret_cast<uint16_t *>(cell) + unit;
            const uint16_t m = (uint16_t)mbits;
            *p = (uint16_t)((*p & ~m) | (uint16_t)nbits);
        }
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
        const E *ks = reinterpret_cast<const E *>(k_row_ptr(st, bh, slot));
        E *kd = reinterpret_cast<E *>(dst_k) + ((size_t)bh * nrows + i) * st.Dk;
        for (int d = threadIdx.x; d < st.Dk; d += blockDim.x) kd[d] = ks[d];
    }
    if (dst_v) {
        const E *vs = reinterpret_cast<const E *>(v_cell_ptr(st, bh, slot));
        E *vd = reinterpret_cast<E *>(dst_v) + ((size_t)bh * nrows + i) * st.Dv;
        const int ub = v_unit_base(slot, st.Dv);
        const int e = v_pos(slot);
        for (int d = threadIdx.x; d < st.Dv; d += blockDim.x) vd[d] = vs[(size_t)(ub + d) * 8 + e];
    }
}

template <int ES>
__global__ void import_fp_kernel(Store st, const char *src_k, const char *src_v, int nrows) {
    const int bh = blockIdx.y;
    const int slot = blockIdx.x;
    using E = typename std::conditional<ES == 2, uint16_t, uint32_t>::type;
    const E *ks = reinterpret_cast<const E *>(src_k) + ((size_t)bh * nrows + slot) * st.Dk;
    E *kd = reinterpret_cast<E *>(const_cast<char *>(k_row_ptr(st, bh, slot)));
    for (int d = threadIdx.x; d < st.Dk; d += blockDim.x) kd[d] = ks[d];
    const E *vs = reinterpret_cast<const E *>(src_v) + ((size_t)bh * nrows + slot) * st.Dv;
    E *vd = reinterpret_cast<E *>(const_cast<char *>(v_cell_ptr(st, bh, slot)));
    const int ub = v_unit_base(slot, st.Dv);
    const int e = v_pos(slot);
    for (int d = threadIdx.x; d < st.Dv; d += blockDim.x) vd[(size_t)(ub + d) * 8 + e] = vs[d];
}

template <int ES>
__global__ void compact_fp_kernel(Store src, Runs runs, Store dst, int nrows) {
    const int bh = blockIdx.y;
    const int i = blockIdx.x;
    const int slot = row_to_slot(runs, i);
    if (slot < 0) return;
    using E = typename std::conditional<ES == 2, uint16_t, uint32_t>::type;
    const E *ks = reinterpret_cast<const E *>(k_row_ptr(src, bh, slot));
    E *kd = reinterpret_cast<E *>(const_cast<char *>(k_row_ptr(dst, bh, i)));
    for (int d = threadIdx.x; d < src.Dk; d += blockDim.x) kd[d] = ks[d];
    const E *vs = reinterpret_cast<const E *>(v_cell_ptr(src, bh, slot));
    E *vd = reinterpret_cast<E *>(const_cast<char *>(v_cell_ptr(dst, bh, i)));
    const int ubs = v_unit_base(slot, src.Dv), es = v_pos(slot);
    const int ubd = v_unit_base(i, src.Dv), ed = v_pos(i);
    for (int d = threadIdx.x; d < src.Dv; d += blockDim.x) vd[(size_t)(ubd + d) * 8 + ed] = vs[(size_t)(ubs + d) * 8 + es];
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
        const int W = st.Dv / per;
        const char *cell = v_cell_ptr(st, bh, slot);
        const int ub = v_unit_base(slot, st.Dv), e = v_pos(slot);
        uint32_t *d = reinterpret_cast<uint32_t *>(dst) + ((size_t)bh * nrows + slot) * W;
        for (int w = threadIdx.x; w < W; w += blockDim.x) {
            uint32_t word = 0;
            for (int i = 0; i < per; ++i) word |= read_v_code<BITS>(cell, ub + w * per + i, e) << (i * BITS);
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

// grid (32-token blocks, BH): dense reference arrays into slots [0, nrows)
template <int BITS>
__global__ void import_quant_kernel(Store st, const uint32_t *kw, const char *ks, const char *kb,
                                    const uint32_t *vw, const char *vs, const char *vb, int nrows) {
    const int bh = blockIdx.y;
    const int blk = blockIdx.x;
    const int lo = blk * 32, hi = min(nrows, lo + 32);
    const int es = st.es;
    constexpr int per = 32 / BITS;
    const int Wk = st.Dk / per, Wv = st.Dv / per, Gk = st.Dk / st.gs, Gv = st.Dv / st.gs;
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
    const int blk_in_page = (lo & (PAGE - 1)) >> 5;
    const int units = 4 * st.Dv;
    for (int u = threadIdx.x; u < units; u += blockDim.x) {
        const int j = u / st.Dv, d = u - j * st.Dv;
        uint64_t nbits = 0;
        for (int e = 0; e < 8; ++e) {
            const int slot = lo + 4 * j + (e & 3) + 16 * (e >> 2);
            if (slot < hi) {
                const uint32_t word = vw[((size_t)bh * nrows + slot) * Wv + d / per];
                nbits |= (uint64_t)((word >> ((d % per) * BITS)) & ((1u << BITS) - 1u)) << (e * BITS);
            }
        }
        const int unit = (blk_in_page * 4 + j) * st.Dv + d;
        if (BITS == 4) reinterpret_cast<uint32_t *>(cell)[unit] = (uint32_t)nbits;
        else if (BITS == 8) reinterpret_cast<uint64_t *>(cell)[unit] = nbits;
        else reinterpret_cast<uint16_t *>(cell)[unit] = (uint16_t)nbits;
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
    constexpr int per = 32 / BITS;
    const int W = D / per, G = D / gs;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        const uint32_t c = (wq[row * W + d / per] >> ((d % per) * BITS)) & ((1u << BITS) - 1u);
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
        else { if ((DTV) == 0) { CALL(0, 2); } else if ((DTV) == 1) { CALL(1, 2); } else { CALL(2, 2); } } \
    } while (0)

hipError_t launch_append_fp(const Store &st, const void *keys, const void *values, int L, int src0,
                            int slot0, int n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    dim3 grid(n, st.BH), block(128);
    if (st.es == 2)
        hipLaunchKernelGGL(append_fp_kernel<2>, grid, block, 0, s, st, (const char *)keys, (const char *)values, L, src0, slot0);
    else
        hipLaunchKernelGGL(append_fp_kernel<4>, grid, block, 0, s, st, (const char *)keys, (const char *)values, L, src0, slot0);
    return hipGetLastError();
}

hipError_t launch_append_quant(const Store &st, const void *keys, const void *values, int L, int src0,
                               int slot0, int n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    const int nblk = ((slot0 + n - 1) >> 5) - (slot0 >> 5) + 1;
    dim3 grid(nblk, st.BH), block(256);
    const size_t lds = (size_t)32 * st.Dv;
#define CALL(DT, BITS)                                                                           \
    hipLaunchKernelGGL((append_quant_kernel<DT, BITS>), grid, block, lds, s, st, (const char *)keys, \
                       (const char *)values, L, src0, slot0, n)
    KV_DISPATCH_DT_BITS(st.dtype, st.bits, CALL);
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
    if (st.bits == 4) hipLaunchKernelGGL(export_quant_kernel<4>, grid, block, 0, s, st, which, nrows, (char *)dst);
    else if (st.bits == 8) hipLaunchKernelGGL(export_quant_kernel<8>, grid, block, 0, s, st, which, nrows, (char *)dst);
    else hipLaunchKernelGGL(export_quant_kernel<2>, grid, block, 0, s, st, which, nrows, (char *)dst);
    return hipGetLastError();
}

hipError_t launch_import_quant(const Store &st, const void *const srcs[6], int nrows, hipStream_t s) {
    if (nrows <= 0) return hipSuccess;
    dim3 grid((nrows + 31) / 32, st.BH), block(256);
#define IMP(BITS)                                                                                     \
    hipLaunchKernelGGL(import_quant_kernel<BITS>, grid, block, 0, s, st, (const uint32_t *)srcs[0],   \
                       (const char *)srcs[1], (const char *)srcs[2], (const uint32_t *)srcs[3],       \
                       (const char *)srcs[4], (const char *)srcs[5], nrows)
    if (st.bits == 4) IMP(4); else if (st.bits == 8) IMP(8); else IMP(2);
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

hipError_t launch_mask_materialize(const kvhip_mask_plan_t &plan, uint8_t *dst, hipStream_t s) {
    if (plan.cols <= 0) return hipSuccess;
    dim3 grid((plan.cols + 255) / 256, plan.rolled ? 1 : (plan.rows < 1024 ? plan.rows : 1024)), block(256);
    hipLaunchKernelGGL(mask_materialize_kernel, grid, block, 0, s, plan, dst);
    return hipGetLastError();
}

}  // namespace kvhip
