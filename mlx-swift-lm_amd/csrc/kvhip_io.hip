// Append (full precision and quantize-on-append), import/export between the
// page layout and the reference's dense array layout, ring-order gather, and
// the standalone affine quantizer.
#include "kvhip_quant_tile.hpp"

namespace kvhip {

namespace {

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

// The same for 16-bit dtypes and head sizes that are multiples of 8, in whole tiles and 16-byte pieces: a thread forms
// eight adjacent elements of a K row, or one column's values for eight adjacent tokens, which is one 16-byte chunk of
// the interleaved full-precision tile; consecutive threads write consecutive chunks.  grid (tiles, BH, 2): K and V of a
// tile are separate workgroups; a thread requests the codes and (scale, bias) pairs of up to four chunks before it
// converts the first.  Eight codes lie inside two adjacent dwords for every code width (a V tile row's octet of
// tokens likewise, in the order v_bitpos gives).  Rows past the cache's length in the last tile come out as
// whatever their slots hold (zeros, or rows trimmed earlier): finite values nobody presents.
template <int DT> __device__ __forceinline__ void pair_of(uint32_t raw, float &sc, float &bi) {
    if (DT == 0) {
        sc = (float)__builtin_bit_cast(_Float16, (uint16_t)raw);
        bi = (float)__builtin_bit_cast(_Float16, (uint16_t)(raw >> 16));
    } else {
        sc = __uint_as_float(raw << 16);
        bi = __uint_as_float(raw & 0xffff0000u);
    }
}
// `dst_pt` non-null: the destination is scratch whose page p lies at `page0` + p * (sk, sv) and whose page table
// `dst_pt` is still unwritten -- the first workgroup writes its `pages` entries for the kernels that follow, and
// nobody here reads them.
template <int DT, int BITS>
__global__ void __launch_bounds__(256) dequant_tiles16_kernel(Store q, Store dst, PageEntry *dst_pt, int pages, PageEntry page0, size_t sk, size_t sv) {
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    constexpr uint32_t M = (1u << BITS) - 1u;
    constexpr int NB = 4;  // chunks in flight per thread
    const int bh = blockIdx.y, lo = blockIdx.x * TILE;
    auto pack = [](float a, float b) { return DT == 0 ? pk_h2(a, b) : pk_bf2(a, b); };
    if (dst_pt != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {
        for (int p = threadIdx.x; p < pages; p += 256) {
            PageEntry e;
            e.k = page0.k + (size_t)p * sk;
            e.v = page0.v + (size_t)p * sv;
            dst_pt[p] = e;
        }
    }
    const PageEntry de = dst_pt != nullptr ? PageEntry{page0.k + (size_t)(lo >> PAGE_SHIFT) * sk, nullptr, page0.v + (size_t)(lo >> PAGE_SHIFT) * sv, nullptr}
                                           : dst.pt[lo >> PAGE_SHIFT];
    if (blockIdx.z == 0) {
        char *kdst = de.k + (size_t)bh * dst.k_cell + kfp_off(dst, lo, 0);
        const int items = (q.Dk / 8) * TILE, last = (int)q.k_row / 4 - 1;
        for (int base = threadIdx.x; base < items; base += 256 * NB) {
            uint32_t w0[NB], w1[NB], sb[NB];
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int item = base + 256 * u;
                if (item < items) {
                    const int c = item >> 6, slot = lo + (item & 63), wi = (8 * c * BITS) >> 5;
                    const uint32_t *row = reinterpret_cast<const uint32_t *>(k_row_ptr(q, bh, slot));
                    w0[u] = row[wi];
                    w1[u] = row[min(wi + 1, last)];
                    sb[u] = reinterpret_cast<const uint32_t *>(ksb_row_ptr(q, bh, slot))[(8 * c) / q.gs];
                }
            }
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                const int item = base + 256 * u;
                if (item < items) {
                    const int off = ((item >> 6) * 8 * BITS) & 31;
                    const uint64_t bits = (((uint64_t)w1[u] << 32) | w0[u]) >> off;
                    float sc, bi, x[8];
                    pair_of<DT>(sb[u], sc, bi);
#pragma unroll
                    for (int j = 0; j < 8; ++j) x[j] = __fadd_rn(__fmul_rn(sc, (float)((uint32_t)(bits >> (j * BITS)) & M)), bi);
                    *reinterpret_cast<u4v *>(kdst + (size_t)item * 16) = u4v{pack(x[0], x[1]), pack(x[2], x[3]), pack(x[4], x[5]), pack(x[6], x[7])};
                }
            }
        }
        return;
    }
    const char *vcell = v_cell_ptr(q, bh, lo);
    char *vdst = de.v + (size_t)bh * dst.v_cell + vfp_off(dst, lo, 0);
    const int items = 8 * q.Dv, last = TILE * BITS / 32 - 1;
    for (int base = threadIdx.x; base < items; base += 256 * NB) {
        uint32_t w0[NB], w1[NB], sb[NB][8];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int item = base + 256 * u;
            if (item < items) {
                const int tc = item / q.Dv, d = item - tc * q.Dv, wi = v_bitpos<BITS>(8 * tc) >> 5;
                const uint32_t *row = reinterpret_cast<const uint32_t *>(vcell + v_row_off(q, lo, d));
                w0[u] = row[wi];
                w1[u] = row[min(wi + 1, last)];
                const int g = d / q.gs;
#pragma unroll
                for (int j = 0; j < 8; ++j) sb[u][j] = reinterpret_cast<const uint32_t *>(vsb_row_ptr(q, bh, lo + 8 * tc + j))[g];
            }
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int item = base + 256 * u;
            if (item < items) {
                const int tc = item / q.Dv, first = v_bitpos<BITS>(8 * tc) & ~31;
                const uint64_t bits = ((uint64_t)w1[u] << 32) | w0[u];
                float x[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    float sc, bi;
                    pair_of<DT>(sb[u][j], sc, bi);
                    x[j] = __fadd_rn(__fmul_rn(sc, (float)((uint32_t)(bits >> (v_bitpos<BITS>(8 * tc + j) - first)) & M)), bi);
                }
                *reinterpret_cast<u4v *>(vdst + (size_t)item * 16) = u4v{pack(x[0], x[1]), pack(x[2], x[3]), pack(x[4], x[5]), pack(x[6], x[7])};
            }
        }
    }
}

// The same for head sizes that are multiples of 32, by units of 32 codes (4 BITS bytes: whole dwords for every code
// width).  A thread loads one unit -- the units of a tile's K rows, and of its V tile rows, are one contiguous run, so
// the loads of a workgroup are too --, converts it and writes four 16-byte chunks of the interleaved full-precision
// tile; for each of the four, the threads of a wavefront write runs of 256 bytes (K: sixteen tokens of one chunk
// column) or 512 bytes (V: thirty-two columns of one token octet).  A K unit has one (scale, bias) pair, loaded with
// it; a V unit needs the pairs of its 32 tokens, which the workgroup stages in LDS once ([group][token]).
// code j (0..31) of a unit held in N dwords, at unit-relative bit `pos` (constant once unrolled)
template <int BITS, int N> __device__ __forceinline__ uint32_t unit_code(const uint32_t (&w)[N], int pos) {
    const int wi = pos >> 5, sh = pos & 31;
    uint32_t v = w[wi] >> sh;
    if (sh + BITS > 32) v |= w[wi + 1 < N ? wi + 1 : wi] << ((32 - sh) & 31);
    return v & ((1u << BITS) - 1u);
}
template <int DT, int BITS>
__global__ void __launch_bounds__(256) dequant_units_kernel(Store q, Store dst, PageEntry *dst_pt, int pages, PageEntry page0, size_t sk, size_t sv) {
    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
    const int bh = blockIdx.y, lo = blockIdx.x * TILE;
    auto pack = [](float a, float b) { return DT == 0 ? pk_h2(a, b) : pk_bf2(a, b); };
    if (dst_pt != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {
        for (int p = threadIdx.x; p < pages; p += 256) {
            PageEntry e;
            e.k = page0.k + (size_t)p * sk;
            e.v = page0.v + (size_t)p * sv;
            dst_pt[p] = e;
        }
    }
    const PageEntry de = dst_pt != nullptr ? PageEntry{page0.k + (size_t)(lo >> PAGE_SHIFT) * sk, nullptr, page0.v + (size_t)(lo >> PAGE_SHIFT) * sv, nullptr}
                                           : dst.pt[lo >> PAGE_SHIFT];
    if (blockIdx.z == 0) {
        char *kdst = de.k + (size_t)bh * dst.k_cell + kfp_off(dst, lo, 0);
        const int upr = q.Dk / 32;  // units per row
        const uint32_t *krows = reinterpret_cast<const uint32_t *>(k_row_ptr(q, bh, lo));  // the tile's 64 rows are contiguous
        for (int u = threadIdx.x; u < upr * TILE; u += 256) {
            const int t = u / upr, p = u - t * upr;
            uint32_t w[BITS];
#pragma unroll
            for (int e = 0; e < BITS; ++e) w[e] = krows[(size_t)u * BITS + e];
            float sc, bi;
            pair_of<DT>(reinterpret_cast<const uint32_t *>(ksb_row_ptr(q, bh, lo + t))[(32 * p) / q.gs], sc, bi);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                uint32_t o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float x0 = __fadd_rn(__fmul_rn(sc, (float)unit_code<BITS, BITS>(w, (8 * k + 2 * j) * BITS)), bi);
                    const float x1 = __fadd_rn(__fmul_rn(sc, (float)unit_code<BITS, BITS>(w, (8 * k + 2 * j + 1) * BITS)), bi);
                    o[j] = pack(x0, x1);
                }
                *reinterpret_cast<u4v *>(kdst + ((size_t)(4 * p + k) * TILE + t) * 16) = u4v{o[0], o[1], o[2], o[3]};
            }
        }
        return;
    }
    // V: the pairs of the tile's 64 tokens, [group][token], through LDS
    extern __shared__ uint32_t sbv[];
    const int G = q.Dv / q.gs;
    for (int i = threadIdx.x; i < G * TILE; i += 256) {
        const int t = i / G, g = i - t * G;
        sbv[g * TILE + t] = reinterpret_cast<const uint32_t *>(vsb_row_ptr(q, bh, lo + t))[g];
    }
    __syncthreads();
    const uint32_t *vrows = reinterpret_cast<const uint32_t *>(v_cell_ptr(q, bh, lo) + v_row_off(q, lo, 0));  // Dv rows of 2 BITS dwords
    char *vdst = de.v + (size_t)bh * dst.v_cell + vfp_off(dst, lo, 0);
    for (int u = threadIdx.x; u < 2 * q.Dv; u += 256) {
        const int d = u >> 1, half = u & 1;
        uint32_t w[BITS];
#pragma unroll
        for (int e = 0; e < BITS; ++e) w[e] = vrows[(size_t)u * BITS + e];
        const uint32_t *sb = sbv + (d / q.gs) * TILE + 32 * half;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float s0, b0, s1, b1;
                pair_of<DT>(sb[8 * k + 2 * j], s0, b0);
                pair_of<DT>(sb[8 * k + 2 * j + 1], s1, b1);
                const float x0 = __fadd_rn(__fmul_rn(s0, (float)unit_code<BITS, BITS>(w, v_bitpos<BITS>(8 * k + 2 * j))), b0);
                const float x1 = __fadd_rn(__fmul_rn(s1, (float)unit_code<BITS, BITS>(w, v_bitpos<BITS>(8 * k + 2 * j + 1))), b1);
                o[j] = pack(x0, x1);
            }
            *reinterpret_cast<u4v *>(vdst + ((size_t)(4 * half + k) * q.Dv + d) * 16) = u4v{o[0], o[1], o[2], o[3]};
        }
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
    const bool tiled = quant_tiles_one_launch(st) || quant_tiles_two_sided(st);
    const TileSplit t = tile_split(slot0, n);
    if (!tiled || t.tiles == 0) return launch_append_quant_rows(st, keys, values, L, src0, slot0, n, s, r);
    hipError_t e = launch_append_quant_rows(st, keys, values, L, src0, slot0, t.head, s, r);
    if (e != hipSuccess) return e;
    const int a0 = src0 + t.head, b0 = slot0 + t.head;
    if (st.bits == 4) e = launch_quant_tiles_bits<4, true, false>(st, st, keys, values, L, a0, b0, t.tiles, s, r);
    else if (st.bits == 8) e = launch_quant_tiles_bits<8, true, false>(st, st, keys, values, L, a0, b0, t.tiles, s, r);
    else e = launch_quant_tiles_other(st, keys, values, L, a0, b0, t.tiles, s, r);
    if (e != hipSuccess) return e;
    return launch_append_quant_rows(st, keys, values, L, a0 + t.tiles * TILE, b0 + t.tiles * TILE, t.tail, s, r);
}

hipError_t launch_requant_pages(const Store &src, const Store &st, int rows, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    const int tiles = (rows + TILE - 1) / TILE;
    if (!quant_tiles_one_launch(st) && !quant_tiles_two_sided(st)) {
        dim3 grid(tiles, st.BH), block(256);
        const size_t lds = (size_t)TILE * st.Dv;
#define CALL(DT, BITS) hipLaunchKernelGGL((requant_rows_kernel<DT, BITS>), grid, block, lds, s, st, src, 0, rows)
        KV_DISPATCH_DT_BITS(st.dtype, st.bits, CALL);
#undef CALL
        return hipGetLastError();
    }
    // whole tiles, the last one included: its rows past `rows` hold zeros or rows trimmed earlier, and
    // what they quantize to lies past the new cache's offset, where the next append overwrites it
    const RopeDev none;
    if (st.bits == 4) return launch_quant_tiles_bits<4, true, true>(st, src, nullptr, nullptr, 0, 0, 0, tiles, s, none);
    if (st.bits == 8) return launch_quant_tiles_bits<8, true, true>(st, src, nullptr, nullptr, 0, 0, 0, tiles, s, none);
    return launch_requant_tiles_other(src, st, tiles, s);
}

hipError_t launch_dequant_pages(const Store &q, const Store &dst, int rows, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    dim3 grid((rows + TILE - 1) / TILE, q.BH), block(256);
    if (q.es == 2 && q.Dk % 8 == 0 && q.Dv % 8 == 0) {
        const size_t lds = (size_t)(q.Dv / q.gs) * TILE * 4;
#define CALL(DT, BITS)                                                                                                  \
    do {                                                                                                                \
        if (q.Dk % 32 == 0 && q.Dv % 32 == 0)                                                                           \
            hipLaunchKernelGGL((dequant_units_kernel<(DT == 2 ? 0 : DT), BITS>), dim3(grid.x, grid.y, 2), block, lds, s, q, dst, \
                               (PageEntry *)nullptr, 0, PageEntry(), (size_t)0, (size_t)0);                             \
        else                                                                                                            \
            hipLaunchKernelGGL((dequant_tiles16_kernel<(DT == 2 ? 0 : DT), BITS>), dim3(grid.x, grid.y, 2), block, 0, s, q, dst, \
                               (PageEntry *)nullptr, 0, PageEntry(), (size_t)0, (size_t)0);                             \
    } while (0)
        KV_DISPATCH_DT_BITS(q.dtype, q.bits, CALL);
#undef CALL
        return hipGetLastError();
    }
#define CALL(DT, BITS) hipLaunchKernelGGL((dequant_pages_kernel<DT, BITS>), grid, block, 0, s, q, dst, rows)
    KV_DISPATCH_DT_BITS(q.dtype, q.bits, CALL);
#undef CALL
    return hipGetLastError();
}

// The same into scratch pages whose table the launch writes itself (16-bit dtypes, head sizes that are multiples of 8):
// page p of the scratch at `page0` + p * (sk, sv), `dst.pt` the table to fill, `dst` otherwise only geometry.
hipError_t launch_dequant_scratch(const Store &q, const Store &dst, int rows, int pages, const PageEntry &page0, size_t sk, size_t sv,
                                  hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    if (q.es != 2 || q.Dk % 8 != 0 || q.Dv % 8 != 0) return hipErrorInvalidValue;
    dim3 grid((rows + TILE - 1) / TILE, q.BH, 2), block(256);
    const size_t lds = (size_t)(q.Dv / q.gs) * TILE * 4;
#define CALL(DT, BITS)                                                                                          \
    do {                                                                                                        \
        if (q.Dk % 32 == 0 && q.Dv % 32 == 0)                                                                   \
            hipLaunchKernelGGL((dequant_units_kernel<(DT == 2 ? 0 : DT), BITS>), grid, block, lds, s, q, dst,    \
                               const_cast<PageEntry *>(dst.pt), pages, page0, sk, sv);                          \
        else                                                                                                    \
            hipLaunchKernelGGL((dequant_tiles16_kernel<(DT == 2 ? 0 : DT), BITS>), grid, block, 0, s, q, dst,    \
                               const_cast<PageEntry *>(dst.pt), pages, page0, sk, sv);                          \
    } while (0)
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

// Dense rows of one pitch into dense rows of another: the common prefix of every row is copied, what is left of a
// wider destination row is zero-filled.  (How arrays of a head size the tuned kernels are not built for are widened
// to the size the cache stores, and narrowed again on the way out.)
template <typename U>
__global__ void __launch_bounds__(256) repitch_rows_kernel(U *dst, uint32_t dst_units, const U *src, uint32_t src_units, size_t rows) {
    const size_t total = rows * dst_units;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const size_t row = i / dst_units;
        const uint32_t u = (uint32_t)(i - row * dst_units);
        dst[i] = u < src_units ? src[row * src_units + u] : (U)0;
    }
}

hipError_t launch_repitch_rows(void *dst, size_t dst_pitch, const void *src, size_t src_pitch, size_t rows, hipStream_t s) {
    if (rows == 0 || dst_pitch == 0) return hipSuccess;
    if ((dst_pitch | src_pitch) & 1) return hipErrorInvalidValue;
    const bool words = ((dst_pitch | src_pitch) & 3) == 0;
    const size_t units = rows * (dst_pitch / (words ? 4 : 2));
    const unsigned blocks = (unsigned)std::min<size_t>((units + 255) / 256, 4096);
    if (words)
        hipLaunchKernelGGL(repitch_rows_kernel<uint32_t>, dim3(blocks), dim3(256), 0, s, (uint32_t *)dst, (uint32_t)(dst_pitch / 4),
                           (const uint32_t *)src, (uint32_t)(src_pitch / 4), rows);
    else
        hipLaunchKernelGGL(repitch_rows_kernel<uint16_t>, dim3(blocks), dim3(256), 0, s, (uint16_t *)dst, (uint32_t)(dst_pitch / 2),
                           (const uint16_t *)src, (uint32_t)(src_pitch / 2), rows);
    return hipGetLastError();
}

hipError_t launch_mask_materialize(const kvhip_mask_plan_t &plan, uint8_t *dst, hipStream_t s) {
    if (plan.cols <= 0) return hipSuccess;
    dim3 grid((plan.cols + 255) / 256, plan.rolled ? 1 : (plan.rows < 1024 ? plan.rows : 1024)), block(256);
    hipLaunchKernelGGL(mask_materialize_kernel, grid, block, 0, s, plan, dst);
    return hipGetLastError();
}

}  // namespace kvhip
