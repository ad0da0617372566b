// Attention on the vector ALUs, for the full-precision caches the matrix-core kernels are not built for: float32
// caches, and 16-bit caches of head sizes above 256 (Gemma 4's full-attention layers: 512).  The fused op
// (AttentionUtils.swift:86-93) computes in float32, excluded keys contribute nothing, one rounding at the output.
//
// 2 * rows FMAs per cached element is below what the memory system delivers them at up to 8 query rows per kv head,
// as long as every cached element is read once per workgroup and the loads are whole cache lines.  The interleaved
// page layout gives both:
//   scores   a lane owns one key of a 64-key tile and reads its row as 16-byte chunks (1 KB per wavefront load);
//            the query rows are wave-uniform: scalar operands (float32) or broadcast from LDS;
//   outputs  a lane owns output columns lane, lane + 64, ... and reads the 4 or 8 tokens of a column's 16-byte chunk,
//            the probabilities are broadcast from LDS.
// A workgroup takes RB query rows of one kv head (row = query head of the group * L + position) and one range of
// key tiles; its four wavefronts walk alternate tiles with their own running maximum / sum / accumulators and are
// merged through LDS at the end.  With more than one key range per (kv head, row block) the workgroup writes an
// unnormalised partial and `merge_valu_kernel` finishes the rows.
#include <algorithm>

#include "kvhip_mask.hpp"

namespace kvhip {

namespace {

constexpr int FT = 256;  // threads per workgroup
constexpr int FW = FT / 64;

typedef float kv_f4 __attribute__((ext_vector_type(4)));

// the 4 (float32) or 8 (16-bit) elements of a 16-byte chunk as floats
template <int DT> struct Chunk {
    static constexpr int N = DT == 2 ? 4 : 8;
};
template <int DT> __device__ __forceinline__ void chunk_floats(const kv_u4 w, float (&f)[Chunk<DT>::N]) {
    if constexpr (DT == 2) {
#pragma unroll
        for (int j = 0; j < 4; ++j) f[j] = __uint_as_float(w[j]);
    } else if constexpr (DT == 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f[2 * j] = __uint_as_float(w[j] << 16);
            f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f[2 * j] = __half2float(__ushort_as_half((unsigned short)(w[j] & 0xffffu)));
            f[2 * j + 1] = __half2float(__ushort_as_half((unsigned short)(w[j] >> 16)));
        }
    }
}

// SQ (float32 only): key rows of whole 16-byte chunks (Dk % 4 == 0).  The query rows are then read straight from the
// caller's array: their addresses are wave-uniform, so they arrive through the scalar cache as FMA operands and the LDS
// is left to the probabilities (with the queries broadcast from LDS too, LDS reads and not FMAs bound a prompt chunk).
template <int DT, int RB, int NC, bool SQ>
__global__ void __launch_bounds__(FT)
attend_valu_kernel(AttendArgs a, int tiles_total, int tiles_per_part, int nparts) {
    static_assert(!SQ || DT == 2, "scalar query operands are float32");
    constexpr int N = Chunk<DT>::N;      // elements per 16-byte chunk
    constexpr int PB = (FW > NC ? FW : NC) * RB * 64;
    extern __shared__ __align__(16) float smem[];
    const Store &st = a.st;
    const int nck = (st.Dk + N - 1) / N;         // 16-byte chunks per key row
    float *qs = smem;                            // (not SQ) [RB][nck * N] scaled query rows, zero beyond Dk
    float *ps = qs + (SQ ? 0 : RB * nck * N);    // [FW][RB][64] probabilities of the wavefront's tile; at the end
                                                 // [RB][NC][64] accumulators of the wavefront being merged
    float *bml = ps + PB;                        // [RB][2] its running maximum and sum

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Workgroups are handed to the 8 XCDs in turn, in id order (x fastest).  The row blocks of one kv head and key
    // range read the same keys and values: ids that are congruent modulo 8 are renumbered to be consecutive, so
    // those row blocks run on one XCD, about the same time, and share its L2.
    int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const int total = gridDim.x * gridDim.y * gridDim.z;
    if (gridDim.x > 1 && (total & 7) == 0) lin = (lin & 7) * (total >> 3) + (lin >> 3);
    const int bh = (lin / gridDim.x) % gridDim.y, part = lin / (gridDim.x * gridDim.y);
    const int b = bh / a.Hkv, h = bh % a.Hkv;
    const int r = a.Hq / a.Hkv, R = r * a.L;
    const int row0 = (lin % gridDim.x) * RB;

    for (int i = tid; !SQ && i < RB * nck * N; i += FT) {
        const int ri = i / (nck * N), d = i % (nck * N), rr = row0 + ri;
        float v = 0.f;
        if (rr < R && d < st.Dk) {
            const int hq = h * r + rr / a.L, l = rr % a.L;
            v = Elem<DT>::load(a.q, ((size_t)(b * a.Hq + hq) * a.L + l) * st.Dk + d) * a.scale;
        }
        qs[i] = v;
    }
    __syncthreads();

    float m[RB], lsum[RB], acc[RB][NC];
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        m[i] = -INFINITY;
        lsum[i] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[i][c] = 0.f;
    }
    float *pw = ps + wave * RB * 64;
    int row_hq[RB], row_l[RB];  // query head and position of the workgroup's rows (-1: beyond the last row)
    const float *qrow[RB];      // (SQ) the rows themselves; beyond the last row: the last row again, which nobody keeps
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        const int rr = row0 + i, rc = min(rr, R - 1);
        row_hq[i] = rr < R ? h * r + rr / a.L : -1;
        row_l[i] = rr < R ? rr % a.L : 0;
        qrow[i] = reinterpret_cast<const float *>(a.q) + ((size_t)(b * a.Hq + h * r + rc / a.L) * a.L + rc % a.L) * st.Dk;
    }
    const float post = SQ ? a.scale : 1.f;

    const int t_begin = part * tiles_per_part, t_end = min(tiles_total, t_begin + tiles_per_part);
    // every wavefront makes the same number of trips, so the barriers below are reached by all of them
    for (int t0 = t_begin; t0 < t_end; t0 += FW) {
        const int t = t0 + wave;
        const bool tile_on = t < t_end;
        const int slot0 = t * TILE, slot = slot0 + lane;
        const int row = (tile_on && slot < a.slots) ? slot_to_row(a.runs, slot) : -1;
        const bool valid = row >= 0 && row < a.T;
        // which of the workgroup's rows see this lane's key, and the additive term of a float array mask
        uint32_t keep = 0;
        float add[RB];
#pragma unroll
        for (int i = 0; i < RB; ++i) {
            add[i] = 0.f;
            if (valid && row_hq[i] >= 0 && mask_keep(a.mask, b, row_hq[i], row_l[i], row, a.L, a.T, add[i])) keep |= 1u << i;
        }
        const bool any = __any(keep != 0);  // wave-uniform: a tile nobody sees is not read
        if (any) {
            float s[RB];
#pragma unroll
            for (int i = 0; i < RB; ++i) s[i] = 0.f;
            gptr kt = as_global(k_cell_ptr(st, bh, slot0)) + (size_t)((slot0 & (PAGE - 1)) >> 6) * ((size_t)TILE * st.k_row) + lane * 16;
            constexpr int U = 8;  // chunks requested together
            for (int c0 = 0; c0 < nck; c0 += U) {
                kv_u4 kv[U];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    kv[u] = (c0 + u < nck) ? ld_global<kv_u4>(kt + (size_t)(c0 + u) * (TILE * 16)) : kv_u4{0u, 0u, 0u, 0u};
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (c0 + u < nck) {
                        // columns beyond Dk in the last chunk meet zero query elements; the pages start from
                        // zero and only whole rows are written, so what they hold is finite
                        float kf[N];
                        chunk_floats<DT>(kv[u], kf);
#pragma unroll
                        for (int i = 0; i < RB; ++i) {
#pragma unroll
                            for (int e = 0; e < N / 4; ++e) {
                                const kv_f4 qv = SQ ? *reinterpret_cast<const kv_f4 *>(qrow[i] + (c0 + u) * 4)
                                                    : *reinterpret_cast<const kv_f4 *>(qs + (i * nck + c0 + u) * N + e * 4);
                                s[i] = fmaf(qv.x, kf[4 * e], s[i]);
                                s[i] = fmaf(qv.y, kf[4 * e + 1], s[i]);
                                s[i] = fmaf(qv.z, kf[4 * e + 2], s[i]);
                                s[i] = fmaf(qv.w, kf[4 * e + 3], s[i]);
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                const bool k = (keep >> i) & 1u;
                const float sc = k ? s[i] * post + add[i] : -INFINITY;
                float mx = sc;
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
                const float mn = fmaxf(m[i], mx);
                float p = 0.f;
                if (mn > -INFINITY) {  // wave-uniform
                    const float corr = expf(m[i] - mn);  // exp(-inf) = 0 for a row's first visible tile
                    p = sc > -INFINITY ? expf(sc - mn) : 0.f;
                    lsum[i] = lsum[i] * corr + p;
#pragma unroll
                    for (int c = 0; c < NC; ++c) acc[i][c] *= corr;
                    m[i] = mn;
                }
                pw[i * 64 + lane] = p;
            }
        }
        __syncthreads();
        if (any) {
            gptr vt = as_global(v_cell_ptr(st, bh, slot0)) + (size_t)((slot0 & (PAGE - 1)) >> 6) * ((size_t)TILE * st.Dv * st.es);
#pragma unroll 2
            for (int tc = 0; tc < TILE / N; ++tc) {
                kv_u4 vv[NC];
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const int col = lane + 64 * c;
                    vv[c] = col < st.Dv ? ld_global<kv_u4>(vt + ((size_t)tc * st.Dv + col) * 16) : kv_u4{0u, 0u, 0u, 0u};
                }
                kv_f4 pr[RB][N / 4];
#pragma unroll
                for (int i = 0; i < RB; ++i)
#pragma unroll
                    for (int e = 0; e < N / 4; ++e) pr[i][e] = *reinterpret_cast<const kv_f4 *>(pw + i * 64 + tc * N + e * 4);
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    float vf[N];
                    chunk_floats<DT>(vv[c], vf);
#pragma unroll
                    for (int i = 0; i < RB; ++i) {
#pragma unroll
                        for (int e = 0; e < N / 4; ++e) {
                            acc[i][c] = fmaf(pr[i][e].x, vf[4 * e], acc[i][c]);
                            acc[i][c] = fmaf(pr[i][e].y, vf[4 * e + 1], acc[i][c]);
                            acc[i][c] = fmaf(pr[i][e].z, vf[4 * e + 2], acc[i][c]);
                            acc[i][c] = fmaf(pr[i][e].w, vf[4 * e + 3], acc[i][c]);
                        }
                    }
                }
            }
        }
        __syncthreads();
    }

    // ---- the four wavefronts' states into the first one's, one after the other ---------------------
#pragma unroll
    for (int i = 0; i < RB; ++i) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) lsum[i] += __shfl_xor(lsum[i], off);
    }
    for (int w = 1; w < FW; ++w) {
        if (wave == w) {
#pragma unroll
            for (int i = 0; i < RB; ++i) {
#pragma unroll
                for (int c = 0; c < NC; ++c) ps[(i * NC + c) * 64 + lane] = acc[i][c];
                if (lane == 0) {
                    bml[2 * i] = m[i];
                    bml[2 * i + 1] = lsum[i];
                }
            }
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                const float mw = bml[2 * i], lw = bml[2 * i + 1];
                const float M = fmaxf(m[i], mw);
                const float f0 = m[i] > -INFINITY ? expf(m[i] - M) : 0.f, fw = mw > -INFINITY ? expf(mw - M) : 0.f;
                lsum[i] = lsum[i] * f0 + lw * fw;
#pragma unroll
                for (int c = 0; c < NC; ++c) acc[i][c] = acc[i][c] * f0 + ps[(i * NC + c) * 64 + lane] * fw;
                m[i] = M;
            }
        }
        __syncthreads();
    }
    if (wave != 0) return;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        const int rr = row0 + i;
        if (rr >= R) continue;
        if (nparts == 1) {
            const size_t o = ((size_t)(b * a.Hq + row_hq[i]) * a.L + row_l[i]) * st.Dv;
#pragma unroll
            for (int c = 0; c < NC; ++c)
                if (lane + 64 * c < st.Dv) Elem<DT>::store(a.out, o + lane + 64 * c, lsum[i] > 0.f ? acc[i][c] / lsum[i] : 0.f);
        } else {
            float *dst = a.workspace + ((size_t)(bh * nparts + part) * R + rr) * (st.Dv + 2);
#pragma unroll
            for (int c = 0; c < NC; ++c)
                if (lane + 64 * c < st.Dv) dst[lane + 64 * c] = acc[i][c];
            if (lane == 0) {
                dst[st.Dv] = m[i];
                dst[st.Dv + 1] = lsum[i];
            }
        }
    }
}

// grid (R, BH), four wavefronts: the partials [bh][part][row][Dv + 2] of one query row into its output row (up to 64
// parts: in every wavefront lane p weighs part p, then each thread sums its columns over the parts with independent loads)
template <int DT>
__global__ void __launch_bounds__(FT)
merge_valu_kernel(AttendArgs a, int nparts) {
    __shared__ float ws[FW][64];
    const int rr = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int b = bh / a.Hkv, h = bh % a.Hkv;
    const int r = a.Hq / a.Hkv, R = r * a.L, Dv = a.st.Dv;
    const float *src = a.workspace + ((size_t)bh * nparts * R + rr) * (Dv + 2);
    const size_t pitch = (size_t)R * (Dv + 2);
    const float mp = lane < nparts ? src[lane * pitch + Dv] : -INFINITY;
    const float lp = lane < nparts ? src[lane * pitch + Dv + 1] : 0.f;
    float M = mp;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off));
    const float w = mp > -INFINITY ? expf(mp - M) : 0.f;
    float Lt = lp * w;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) Lt += __shfl_xor(Lt, off);
    ws[wave][lane] = w;
    __syncthreads();
    const int hq = h * r + rr / a.L, l = rr % a.L;
    const size_t o = ((size_t)(b * a.Hq + hq) * a.L + l) * Dv;
    for (int col = tid; col < Dv; col += FT) {
        float A = 0.f;
#pragma unroll 8
        for (int p = 0; p < nparts; ++p) A = fmaf(src[p * pitch + col], ws[wave][p], A);
        Elem<DT>::store(a.out, o + col, Lt > 0.f ? A / Lt : 0.f);
    }
}

struct PlanValu {
    int rb, nc, row_blocks, tiles_total, tiles_per_part, nparts;
    bool sq;
    size_t lds;
};

PlanValu plan_valu(const AttendArgs &a) {
    PlanValu p;
    const int R = (a.Hq / a.Hkv) * a.L;
    p.nc = a.st.Dv <= 64 ? 1 : a.st.Dv <= 128 ? 2 : a.st.Dv <= 256 ? 4 : 8;
    // (16 rows per workgroup would read the keys half as often, but that instance holds one wavefront per SIMD
    // and waits on its scalar loads: measured at 60 % of the 8-row one's rate on prompt chunks)
    p.rb = R <= 4 ? 4 : 8;
    p.tiles_total = (a.slots + TILE - 1) / TILE;
    // a launch that cannot fill the chip even with every key range it may have is bound by latency: row blocks of
    // 4 double its workgroups (one sequence, 2 kv heads of 512, 2 new tokens over 8192 keys: 51 us against 69)
    if (p.rb == 8 && (long)((R + 7) / 8) * a.st.BH * std::min(64, std::max(1, p.tiles_total / FW)) < 256) p.rb = 4;
    p.row_blocks = (R + p.rb - 1) / p.rb;
    p.sq = a.st.dtype == KVHIP_F32 && a.st.Dk % 4 == 0;
    const int n_el = a.st.dtype == KVHIP_F32 ? 4 : 8, nck = (a.st.Dk + n_el - 1) / n_el;
    p.lds = ((p.sq ? 0 : (size_t)p.rb * nck * n_el) + (size_t)std::max(FW, p.nc) * p.rb * 64 + (size_t)p.rb * 2) * sizeof(float);
    // enough workgroups for two per CU; a part keeps at least one tile per wavefront
    const long wgs = (long)p.row_blocks * a.st.BH;
    int n = (int)std::max(1L, std::min<long>(512 / std::max(1L, wgs), p.tiles_total / FW));
    n = std::min(n, 64);
    const size_t per_part = (size_t)a.st.BH * R * (a.st.Dv + 2) * sizeof(float);
    if (a.workspace_cap)
        while (n > 1 && per_part * n > a.workspace_cap) --n;
    p.tiles_per_part = (p.tiles_total + n - 1) / n;
    p.nparts = (p.tiles_total + p.tiles_per_part - 1) / p.tiles_per_part;
    return p;
}

template <int DT, int RB, int NC>
void launch_instance(const AttendArgs &a, const PlanValu &p, hipStream_t s) {
    const dim3 grid(p.row_blocks, a.st.BH, p.nparts), block(FT);
    if constexpr (DT == 2) {
        if (p.sq) {
            hipLaunchKernelGGL((attend_valu_kernel<DT, RB, NC, true>), grid, block, p.lds, s, a, p.tiles_total, p.tiles_per_part, p.nparts);
            return;
        }
    }
    hipLaunchKernelGGL((attend_valu_kernel<DT, RB, NC, false>), grid, block, p.lds, s, a, p.tiles_total, p.tiles_per_part, p.nparts);
}

template <int DT>
hipError_t launch_dt(const AttendArgs &a, const PlanValu &p, hipStream_t s) {
    profile_mark(s, true);
    if (p.nc == 8 && p.rb == 8) launch_instance<DT, 8, 8>(a, p, s);
    else if (p.nc == 8) launch_instance<DT, 4, 8>(a, p, s);
    else if (p.rb == 4) {
        if (p.nc == 1) launch_instance<DT, 4, 1>(a, p, s);
        else if (p.nc == 2) launch_instance<DT, 4, 2>(a, p, s);
        else launch_instance<DT, 4, 4>(a, p, s);
    } else {
        if (p.nc == 1) launch_instance<DT, 8, 1>(a, p, s);
        else if (p.nc == 2) launch_instance<DT, 8, 2>(a, p, s);
        else launch_instance<DT, 8, 4>(a, p, s);
    }
    profile_mark(s, false);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || p.nparts == 1) return e;
    hipLaunchKernelGGL(merge_valu_kernel<DT>, dim3((a.Hq / a.Hkv) * a.L, a.st.BH), dim3(FT), 0, s, a, p.nparts);
    return hipGetLastError();
}

}  // namespace

bool attend_valu_supported(const AttendArgs &a) {
    const Store &s = a.st;
    return s.bits == 0 && s.Dk <= 1024 && s.Dv <= 512 && s.BH <= 65535 && plan_valu(a).lds <= 64 * 1024;
}

bool attend_valu_dequant_first(const AttendArgs &a) {
    const Store &s = a.st;
    if (s.bits == 0) return false;
    if (a.runs.n != 1 || a.runs.row0[0] != 0 || a.runs.phys0[0] != 0) return false;  // the scratch pages hold slots in presented order
    if (s.es == 2 && (s.Dk % 8 != 0 || s.Dv % 8 != 0)) return false;
    AttendArgs fp = a;
    fp.st.bits = 0;
    return attend_valu_supported(fp);
}

size_t attend_valu_workspace(const AttendArgs &a) {
    const PlanValu p = plan_valu(a);
    return p.nparts == 1 ? 0 : (size_t)a.st.BH * p.nparts * (a.Hq / a.Hkv) * a.L * (a.st.Dv + 2) * sizeof(float);
}

hipError_t launch_attend_valu(const AttendArgs &a, hipStream_t s) {
    const PlanValu p = plan_valu(a);
    if (a.st.dtype == KVHIP_F16) return launch_dt<0>(a, p, s);
    if (a.st.dtype == KVHIP_BF16) return launch_dt<1>(a, p, s);
    return launch_dt<2>(a, p, s);
}

}  // namespace kvhip
