// Split-sequence decode attention on the matrix cores (gfx950 MFMA 16x16x32).
//
// One workgroup (4 wavefronts) owns a contiguous span of physical slots of one
// (batch, kv-head) pair and leaves an unnormalised partial (max, sum, out[D]) per
// query row; a second small kernel merges the partials of all spans.  The r*L
// (<= 4) query rows that share a kv head ride in the M dimension of the QK^T
// tile, so K and V are read from HBM exactly once per step.
//
// Per 64-slot tile and wavefront:
//   QK^T   four 16-token sub-tiles are multiplied by four copies of the query
//          block placed in different row groups of the A operand, so that the
//          accumulator of lane l ends up holding the scores of token l for all
//          query rows.  Packed codes become MFMA operands without a dequantize
//          pass: a 4-bit (8-bit) code masked in place is the fp16 subnormal
//          code * 2^-24 (high nibbles: * 2^-20, compensated by queries
//          pre-scaled by 1/16), so q.(scale*code + bias) is evaluated as
//          scale * 2^24 * mfma(q, masked words) + bias * sum(q).
//   softmax online, running maximum per wavefront, rescaling only when a tile
//          raises it.
//   PV     P (times the per-token V scale of the column's group) goes through LDS
//          into the A operand; the octet-transposed V words are the B operand
//          as stored.  V biases are accumulated on the side: sum_t p_t * bias_t.
#include <cstdlib>
#include <vector>

#include "kvhip_mask.hpp"

namespace kvhip {

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
union Op {
    h8 h;
    b8 b;
    uint32_t u[4];
    uint4 v;
};

constexpr int WAVES = 4;
constexpr int TILE = 64;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float TWO24 = 16777216.0f;

// element position inside an 8-element operand chunk for operand slot kk
template <int BITS> __device__ __forceinline__ constexpr int elem_of(int kk) {
    return BITS == 4 ? ((kk >> 1) + 4 * (kk & 1)) : (BITS == 8 ? ((kk & 4) + ((kk >> 1) & 1) + 2 * (kk & 1)) : kk);
}
// operand slot of octet position e (inverse of elem_of)
template <int BITS> __device__ __forceinline__ int slot_of(int e) {
    return BITS == 4 ? (2 * (e & 3) + (e >> 2)) : (BITS == 8 ? ((e & 4) + 2 * (e & 1) + ((e >> 1) & 1)) : e);
}
// slots whose masked value carries an extra factor 16 (high nibbles)
template <int BITS> __device__ __forceinline__ constexpr bool hi_slot(int kk) { return BITS == 4 && (kk & 2); }

template <int BITS> struct Words;  // raw 8-element chunk as loaded
template <> struct Words<4> { uint32_t w; };
template <> struct Words<8> { uint2 w; };
template <> struct Words<0> { uint4 w; };

template <int BITS> __device__ __forceinline__ Op to_operand(const Words<BITS> &x);
template <> __device__ __forceinline__ Op to_operand<4>(const Words<4> &x) {
    Op o;
    const uint32_t w8 = x.w >> 8;
    o.u[0] = x.w & 0x000f000fu;
    o.u[1] = x.w & 0x00f000f0u;
    o.u[2] = w8 & 0x000f000fu;
    o.u[3] = w8 & 0x00f000f0u;
    return o;
}
template <> __device__ __forceinline__ Op to_operand<8>(const Words<8> &x) {
    Op o;
    o.u[0] = x.w.x & 0x00ff00ffu;
    o.u[1] = (x.w.x >> 8) & 0x00ff00ffu;
    o.u[2] = x.w.y & 0x00ff00ffu;
    o.u[3] = (x.w.y >> 8) & 0x00ff00ffu;
    return o;
}
template <> __device__ __forceinline__ Op to_operand<0>(const Words<0> &x) {
    Op o;
    o.v = x.w;
    return o;
}

template <bool BF> __device__ __forceinline__ f4 mfma(const Op &a, const Op &b, f4 c) {
    if (BF) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, c, 0, 0, 0);
}

__device__ __forceinline__ float wave_max(float v) {
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

__device__ __forceinline__ uint16_t f2h_bits(float v) {
    return __builtin_bit_cast(uint16_t, (_Float16)v);
}
__device__ __forceinline__ uint16_t f2bf_bits(float v) { return Elem<1>::bits(v); }

// One tile's worth of raw operand data held in registers.
template <int BITS, int D, int G> struct TileRegs {
    Words<BITS> k[4][D / 32];  // [sub-tile u][step]
    Words<BITS> v[2][D / 16];  // [32-token block][d tile]
    float ks[G], kb[G], vs[G], vb[G];
    int row;                   // presented row of this lane's token, -1 if none
};

// partial layout in the workspace: per (bh, split, query row): m, l, out[D]
template <int D> constexpr int part_stride() { return D + 2; }

template <int BITS, int D, int GS, int DT>
__global__ void __launch_bounds__(WAVES * 64, 2)
decode_kernel(AttendArgs a, int tiles_total, int tiles_per_wg, int nsplit) {
    constexpr bool Q = BITS != 0;
    constexpr bool BF = !Q && DT == 1;  // quantized caches always use fp16 operands
    constexpr int S = D / 32;            // MFMA steps over the head dim
    constexpr int G = Q ? D / GS : 1;    // quantization groups per row
    constexpr int NT = D / 16;           // output column tiles
    const Store &st = a.st;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, j = lane >> 4;
    const int bh = blockIdx.y, split = blockIdx.x;
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int r = a.Hq / a.Hkv;
    const int R = r * a.L;  // query rows sharing this kv head (<= 4)

    __shared__ __attribute__((aligned(16))) uint16_t pbuf[WAVES][2][G][4][TILE];  // [wave][hi/lo][group][row][slot]
    __shared__ float cbuf[WAVES][4][D + 2];

    // ---- query operands: built once per workgroup, kept in LDS ------------------
    // qlds[u][s][lane] is the A operand of sub-tile u at step s: the query block sits in
    // row group u (rows 4u..4u+3) and every other row is zero.
    __shared__ uint4 qlds[4][S][64];
    float qsum[G][4];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) qsum[g][i] = 0.f;
    {
        const int i = n & 3;  // query row this lane feeds
        const int rep = i / a.L, l = i - rep * a.L;
        const size_t qoff = ((size_t)(b * a.Hq + hk * r + rep) * a.L + l) * D;
        const int u = wave;   // wavefront w fills the operands of sub-tile w
        const bool on = (n >> 2) == u && i < R;
#pragma unroll
        for (int s = 0; s < S; ++s) {
            Op base;
#pragma unroll
            for (int w = 0; w < 4; ++w) base.u[w] = 0u;
            if (on) {
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) {
                    const int d = 32 * s + 8 * j + elem_of<BITS>(kk);
                    float qv = Elem<DT>::load(a.q, qoff + d);
                    if (Q) qv = round_dt<DT>(qv * a.scale);
                    const uint16_t hb = BF ? f2bf_bits(qv) : f2h_bits(hi_slot<BITS>(kk) ? qv * 0.0625f : qv);
                    base.u[kk >> 1] |= (uint32_t)hb << (16 * (kk & 1));
                }
            }
            qlds[u][s][lane] = base.v;
        }
        if (Q) {
            // sum of the (rounded, fp16-held) queries per group, for the bias term
#pragma unroll
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
                    float sacc = 0.f;
                    if (ii < R) {
                        const int rep2 = ii / a.L, l2 = ii - rep2 * a.L;
                        const size_t qo = ((size_t)(b * a.Hq + hk * r + rep2) * a.L + l2) * D;
                        for (int d = g * GS + lane; d < (g + 1) * GS; d += 64)
                            sacc += (float)(_Float16)round_dt<DT>(Elem<DT>::load(a.q, qo + d) * a.scale);
                    }
                    qsum[g][ii] = wave_sum(sacc);
                }
        }
    }
    __syncthreads();

    // ---- running state ---------------------------------------------------------
    float m_run[4], l_part[4], bacc[G][4];
    f4 oacc[NT];
#pragma unroll
    for (int i = 0; i < 4; ++i) { m_run[i] = -INFINITY; l_part[i] = 0.f; }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) bacc[g][i] = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t) oacc[t] = f4{0.f, 0.f, 0.f, 0.f};

    const int tile_begin = split * tiles_per_wg;
    const int tile_end = min(tiles_total, tile_begin + tiles_per_wg);
    const float fill = finfo_min_dt(DT);
    // LDS position of this lane's token inside the P staging row
    const int tl = lane & 31;
    const int e_tok = (tl & 3) + ((tl >> 4) << 2);
    const int ppos = (lane & 32) + 8 * ((tl & 15) >> 2) + slot_of<BITS>(e_tok);
    const float vfac = (BITS == 4 && (e_tok & 1)) ? 0.0625f : 1.0f;

    auto load_tile = [&](int tile, TileRegs<BITS, D, G> &t) {
        const int slot0 = tile * TILE;
        // K: sub-tile u, token n, chunk j
        const char *kbase = k_row_ptr(st, bh, slot0 + n);
        constexpr int CH = Q ? BITS : 16;  // bytes per 8-element chunk
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const char *p = kbase + (size_t)u * 16 * st.k_row + (4 * s + j) * CH;
                if constexpr (BITS == 4) t.k[u][s].w = *reinterpret_cast<const uint32_t *>(p);
                else if constexpr (BITS == 8) *reinterpret_cast<uint2 *>(&t.k[u][s].w) = *reinterpret_cast<const uint2 *>(p);
                else *reinterpret_cast<uint4 *>(&t.k[u][s].w) = *reinterpret_cast<const uint4 *>(p);
            }
        // V: block blk, octet j, column tile dt, column n
        const char *vcell = v_cell_ptr(st, bh, slot0);
        const int bip = (slot0 & (PAGE - 1)) >> 5;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int dt = 0; dt < NT; ++dt) {
                const size_t unit = (size_t)((bip + blk) * 4 + j) * D + 16 * dt + n;
                const char *p = vcell + unit * CH;
                if constexpr (BITS == 4) t.v[blk][dt].w = *reinterpret_cast<const uint32_t *>(p);
                else if constexpr (BITS == 8) *reinterpret_cast<uint2 *>(&t.v[blk][dt].w) = *reinterpret_cast<const uint2 *>(p);
                else *reinterpret_cast<uint4 *>(&t.v[blk][dt].w) = *reinterpret_cast<const uint4 *>(p);
            }
        const int slot = slot0 + lane;
        if (Q) {
            const char *ksb = ksb_row_ptr(st, bh, slot);
            const char *vsb = vsb_row_ptr(st, bh, slot);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                t.ks[g] = Elem<DT>::load(ksb, 2 * g);
                t.kb[g] = Elem<DT>::load(ksb, 2 * g + 1);
                t.vs[g] = Elem<DT>::load(vsb, 2 * g);
                t.vb[g] = Elem<DT>::load(vsb, 2 * g + 1);
            }
        }
        const int row = slot < a.slots ? slot_to_row(a.runs, slot) : -1;
        t.row = (row >= 0 && row < a.T) ? row : -1;
    };

    auto compute_tile = [&](const TileRegs<BITS, D, G> &t) {
        // ---- scores -------------------------------------------------------------
        f4 sacc[G];
#pragma unroll
        for (int g = 0; g < G; ++g) sacc[g] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const int g = Q ? (32 * s) / GS : 0;
                Op qa;
                qa.v = qlds[u][s][lane];
                sacc[g] = mfma<BF>(qa, to_operand<BITS>(t.k[u][s]), sacc[g]);
            }
        float sc[4];
        const bool live = t.row >= 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float s_;
            if (Q) {
                s_ = 0.f;
#pragma unroll
                for (int g = 0; g < G; ++g) s_ += (t.ks[g] * TWO24) * sacc[g][i] + t.kb[g] * qsum[g][i];
                s_ = round_dt<DT>(s_);
            } else {
                s_ = sacc[0][i] * a.scale;
            }
            if (live && i < R && a.mask.mode != KVHIP_MASK_NONE) {
                const int rep = i / a.L, l = i - rep * a.L;
                float add;
                const bool keep = mask_keep(a.mask, b, hk * r + rep, l, t.row, a.L, a.T, add);
                if (Q) {
                    if (!keep) s_ = fill;
                    else if (a.mask.mode == KVHIP_MASK_ARRAY && a.mask.dtype != KVHIP_BOOL) s_ = round_dt<DT>(s_ + add);
                } else {
                    s_ = keep ? s_ + add : -INFINITY;
                }
            }
            sc[i] = live ? s_ : -INFINITY;
        }
        // ---- online softmax: raise the running maximum only when a tile exceeds it
        bool need = false;
#pragma unroll
        for (int i = 0; i < 4; ++i) need = need || (sc[i] > m_run[i]);
        if (__any(need)) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float mn = fmaxf(m_run[i], wave_max(sc[i]));
                const float alpha = (mn == -INFINITY) ? 1.f : exp2f((m_run[i] - mn) * LOG2E);
                m_run[i] = mn;
                l_part[i] *= alpha;
#pragma unroll
                for (int g = 0; g < G; ++g) bacc[g][i] *= alpha;
#pragma unroll
                for (int tt = 0; tt < NT; ++tt) oacc[tt][i] *= alpha;
            }
        }
        float p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            p[i] = (sc[i] == -INFINITY) ? 0.f : exp2f((sc[i] - m_run[i]) * LOG2E);
            l_part[i] += p[i];
        }
        // ---- stage P (x per-token V scale) into LDS in A-operand order --------------
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (Q) {
                    bacc[g][i] += p[i] * t.vb[g];
                    pbuf[wave][0][g][i][ppos] = f2h_bits(p[i] * (t.vs[g] * vfac));
                } else if (BF) {
                    const uint16_t hi = f2bf_bits(p[i]);
                    const float rest = p[i] - __uint_as_float((uint32_t)hi << 16);
                    pbuf[wave][0][g][i][ppos] = hi;
                    pbuf[wave][1][g][i][ppos] = f2bf_bits(rest);
                } else {
                    pbuf[wave][0][g][i][ppos] = f2h_bits(p[i]);
                }
            }
        __builtin_amdgcn_wave_barrier();
        // ---- out += P . V ---------------------------------------------------------------
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            Op pa[G], pl[G];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                pa[g].v = *reinterpret_cast<const uint4 *>(&pbuf[wave][0][g][n & 3][blk * 32 + 8 * j]);
                if (BF) pl[g].v = *reinterpret_cast<const uint4 *>(&pbuf[wave][1][g][n & 3][blk * 32 + 8 * j]);
            }
#pragma unroll
            for (int dt = 0; dt < NT; ++dt) {
                const int g = Q ? (16 * dt) / GS : 0;
                const Op vb_ = to_operand<BITS>(t.v[blk][dt]);
                oacc[dt] = mfma<BF>(pa[g], vb_, oacc[dt]);
                if (BF) oacc[dt] = mfma<BF>(pl[g], vb_, oacc[dt]);
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    // ---- main loop: this wavefront takes every WAVES-th tile of the span, one tile
    // of loads in flight ahead of the arithmetic
    // (variants whose tile does not fit twice in the register file run single-buffered
    // and lean on the second resident wavefront to cover the load latency)
    constexpr bool PREFETCH = !(D == 128 && (BITS == 8 || G > 2));
    if constexpr (PREFETCH) {
        TileRegs<BITS, D, G> bufA, bufB;
        int tile = tile_begin + wave;
        if (tile < tile_end) load_tile(tile, bufA);
        while (tile < tile_end) {
            const int next = tile + WAVES;
            if (next < tile_end) load_tile(next, bufB);
            compute_tile(bufA);
            tile = next;
            if (tile >= tile_end) break;
            const int next2 = tile + WAVES;
            if (next2 < tile_end) load_tile(next2, bufA);
            compute_tile(bufB);
            tile = next2;
        }
    } else {
        TileRegs<BITS, D, G> buf;
        for (int tile = tile_begin + wave; tile < tile_end; tile += WAVES) {
            load_tile(tile, buf);
            compute_tile(buf);
        }
    }

    // ---- wavefront partial -> LDS ---------------------------------------------------
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        l_part[i] = wave_sum(l_part[i]);
#pragma unroll
        for (int g = 0; g < G; ++g) bacc[g][i] = wave_sum(bacc[g][i]);
    }
    if (j == 0) {
#pragma unroll
        for (int dt = 0; dt < NT; ++dt) {
            const int g = Q ? (16 * dt) / GS : 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float o = oacc[dt][i];
                if (Q) o = o * TWO24 + bacc[g][i];
                cbuf[wave][i][16 * dt + n] = o;
            }
        }
    }
    if (lane < 4) {
        cbuf[wave][lane][D] = m_run[lane];
        cbuf[wave][lane][D + 1] = l_part[lane];
    }
    __syncthreads();
    // ---- merge the 4 wavefronts, write the span's partial ------------------------------
    float *part = a.workspace + ((size_t)bh * nsplit + split) * 4 * (D + 2);
    for (int idx = threadIdx.x; idx < 4 * (D + 2); idx += WAVES * 64) {
        const int i = idx / (D + 2), c = idx - i * (D + 2);
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, cbuf[w][i][D]);
        float v;
        if (c == D) {
            v = mx;
        } else {
            v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) {
                const float mw = cbuf[w][i][D];
                const float wgt = (mw == -INFINITY) ? 0.f : exp2f((mw - mx) * LOG2E);
                v += wgt * cbuf[w][i][c];
            }
        }
        part[idx] = v;
    }
}

// grid (R, BH): merge the span partials of one query row and write the output row
template <int D, int DT>
__global__ void __launch_bounds__(D)
combine_kernel(AttendArgs a, int nsplit) {
    const int i = blockIdx.x, bh = blockIdx.y;
    const int b = bh / a.Hkv, hk = bh - b * a.Hkv;
    const int r = a.Hq / a.Hkv;
    const int rep = i / a.L, l = i - rep * a.L;
    const float *part = a.workspace + (size_t)bh * nsplit * 4 * (D + 2) + (size_t)i * (D + 2);
    const int d = threadIdx.x;
    float mx = -INFINITY;
    for (int s = 0; s < nsplit; ++s) mx = fmaxf(mx, part[(size_t)s * 4 * (D + 2) + D]);
    float num = 0.f, den = 0.f;
    for (int s = 0; s < nsplit; ++s) {
        const float *p = part + (size_t)s * 4 * (D + 2);
        const float mw = p[D];
        const float w = (mw == -INFINITY) ? 0.f : exp2f((mw - mx) * LOG2E);
        num += w * p[d];
        den += w * p[D + 1];
    }
    const float o = den > 0.f ? num / den : 0.f;
    Elem<DT>::store(a.out, ((size_t)(b * a.Hq + hk * r + rep) * a.L + l) * D + d, o);
}

struct Plan {
    int tiles_total, tiles_per_wg, nsplit;
};

Plan plan_for(const AttendArgs &a) {
    Plan p;
    p.tiles_total = (a.slots + TILE - 1) / TILE;
    const int BH = a.st.BH;
    // enough workgroups to fill 256 CUs several times over; a span is a multiple of
    // WAVES tiles so every wavefront of a workgroup gets the same share
    int want = (256 * 16 + BH - 1) / BH;
    int per = (p.tiles_total + want - 1) / want;
    if (const char *e = getenv("KVHIP_DECODE_TILES")) per = atoi(e);
    per = per < WAVES ? WAVES : per;
    per = (per + WAVES - 1) / WAVES * WAVES;
    p.tiles_per_wg = per;
    p.nsplit = (p.tiles_total + per - 1) / per;
    return p;
}

}  // namespace

namespace {
bool g_profile = false;
std::vector<hipEvent_t> g_events;  // begin/end pairs
}  // namespace

void profile_enable(bool on) { g_profile = on; }

void profile_mark(hipStream_t s, bool) {
    if (!g_profile) return;
    hipEvent_t e;
    if (hipEventCreate(&e) != hipSuccess) return;
    (void)hipEventRecord(e, s);
    g_events.push_back(e);
}

hipError_t profile_read(int *launches, double *total_ms) {
    *launches = 0;
    *total_ms = 0.0;
    for (size_t i = 0; i + 1 < g_events.size(); i += 2) {
        hipError_t e = hipEventSynchronize(g_events[i + 1]);
        if (e != hipSuccess) return e;
        float ms = 0.f;
        e = hipEventElapsedTime(&ms, g_events[i], g_events[i + 1]);
        if (e != hipSuccess) return e;
        *total_ms += ms;
        *launches += 1;
    }
    for (hipEvent_t ev : g_events) (void)hipEventDestroy(ev);
    g_events.clear();
    return hipSuccess;
}

bool attend_decode_supported(const AttendArgs &a) {
    const Store &s = a.st;
    if (s.dtype != KVHIP_F16 && s.dtype != KVHIP_BF16) return false;
    if (s.Dk != s.Dv) return false;
    const int R = (a.Hq / a.Hkv) * a.L;
    if (R > 4) return false;
    if (s.bits == 0) return false;  // full-precision caches: generic kernel for now
    if (s.bits != 4 && s.bits != 8) return false;
    if (s.Dk != 64 && s.Dk != 128) return false;
    return s.gs == 32 || s.gs == 64 || (s.gs == 128 && s.Dk == 128);
}

size_t attend_decode_workspace(const AttendArgs &a) {
    const Plan p = plan_for(a);
    return (size_t)a.st.BH * p.nsplit * 4 * (a.st.Dk + 2) * sizeof(float);
}

hipError_t launch_attend_decode(const AttendArgs &a, hipStream_t s) {
    const Plan p = plan_for(a);
    const Store &st = a.st;
    dim3 grid(p.nsplit, st.BH), block(WAVES * 64);
    const int R = (a.Hq / a.Hkv) * a.L;
#define DEC(BITS, D, GS, DT)                                                                              \
    do {                                                                                                  \
        profile_mark(s, true);                                                                            \
        hipLaunchKernelGGL((decode_kernel<BITS, D, GS, DT>), grid, block, 0, s, a, p.tiles_total,         \
                           p.tiles_per_wg, p.nsplit);                                                     \
        profile_mark(s, false);                                                                           \
        hipLaunchKernelGGL((combine_kernel<D, DT>), dim3(R, st.BH), dim3(D), 0, s, a, p.nsplit);   \
    } while (0)
#define DEC_DT(BITS, D, GS)                      \
    do {                                         \
        if (st.dtype == KVHIP_F16) DEC(BITS, D, GS, 0); \
        else DEC(BITS, D, GS, 1);                \
    } while (0)
#define DEC_Q(BITS)                                               \
    do {                                                          \
        if (st.Dk == 64) {                                        \
            if (st.gs == 32) DEC_DT(BITS, 64, 32);                \
            else DEC_DT(BITS, 64, 64);                            \
        } else {                                                  \
            if (st.gs == 32) DEC_DT(BITS, 128, 32);               \
            else if (st.gs == 64) DEC_DT(BITS, 128, 64);          \
            else DEC_DT(BITS, 128, 128);                          \
        }                                                         \
    } while (0)
    if (st.bits == 4) DEC_Q(4);
    else if (st.bits == 8) DEC_Q(8);
    else return hipErrorNotSupported;
#undef DEC_Q
#undef DEC_DT
#undef DEC
    return hipGetLastError();
}

}  // namespace kvhip
