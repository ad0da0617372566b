// Attention over float32 caches (AttentionUtils.swift:86-93 with float32 keys, values and queries:
// the fused op computes in float32, excluded keys contribute nothing, the output is float32).
//
// The matrix cores take 16-bit operands, so float32 rows stay on the vector ALUs: 2 * rows FMAs per cached
// element is far below what the memory system delivers them at, as long as every cached element is read
// once per workgroup and the loads are whole cache lines.  The interleaved page layout gives both:
//   scores   a lane owns one key of a 64-key tile and reads its row as 16-byte chunks (1 KB per wavefront load),
//            the query rows are broadcast from LDS;
//   outputs  a lane owns output columns lane, lane + 64, ... and reads 4 tokens of a column per 16-byte load,
//            the probabilities are broadcast from LDS.
// A workgroup takes RB query rows of one kv head (row = query head of the group * L + position) and one range of
// key tiles; its four wavefronts walk alternate tiles with their own running maximum / sum / accumulators and are
// merged through LDS at the end.  With more than one key range per (kv head, row block) the workgroup writes an
// unnormalised partial and `merge_f32_kernel` finishes the rows.
#include <algorithm>

#include "kvhip_mask.hpp"

namespace kvhip {

namespace {

constexpr int FT = 256;  // threads per workgroup
constexpr int FW = FT / 64;

typedef float kv_f4 __attribute__((ext_vector_type(4)));

// SQ: key rows of whole 16-byte chunks (Dk % 4 == 0).  The query rows are then read straight from the caller's array:
// their addresses are wave-uniform, so they arrive through the scalar cache as FMA operands and the LDS is left
// to the probabilities (with the queries broadcast from LDS too, LDS reads and not FMAs bound a prompt chunk).
template <int RB, int NC, bool SQ>
__global__ void __launch_bounds__(FT)
attend_f32_kernel(AttendArgs a, int tiles_total, int tiles_per_part, int nparts) {
    extern __shared__ __align__(16) float smem[];
    const Store &st = a.st;
    const int nck = (st.Dk + 3) >> 2;            // 16-byte chunks per key row
    float *qs = smem;                            // (not SQ) [RB][nck * 4] scaled query rows, zero beyond Dk
    float *ps = qs + (SQ ? 0 : RB * nck * 4);    // [FW][RB][64] probabilities of the wavefront's tile
    float *wacc = ps + FW * RB * 64;             // [FW][RB][64 * NC] accumulators at the end
    float *wml = wacc + FW * RB * 64 * NC;       // [FW][RB][2] running maximum, sum

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

    for (int i = tid; !SQ && i < RB * nck * 4; i += FT) {
        const int ri = i / (nck * 4), d = i % (nck * 4), rr = row0 + ri;
        float v = 0.f;
        if (rr < R && d < st.Dk) {
            const int hq = h * r + rr / a.L, l = rr % a.L;
            v = reinterpret_cast<const float *>(a.q)[((size_t)(b * a.Hq + hq) * a.L + l) * st.Dk + d] * a.scale;
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
                kv_f4 kv[U];
#pragma unroll
                for (int u = 0; u < U; ++u)
                    kv[u] = (c0 + u < nck) ? ld_global<kv_f4>(kt + (size_t)(c0 + u) * (TILE * 16)) : kv_f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (c0 + u < nck) {
                        // columns beyond Dk in the last chunk meet zero query elements; the pages start from
                        // zero and only whole rows are written, so what they hold is finite
#pragma unroll
                        for (int i = 0; i < RB; ++i) {
                            const kv_f4 qv = SQ ? *reinterpret_cast<const kv_f4 *>(qrow[i] + (c0 + u) * 4)
                                                : *reinterpret_cast<const kv_f4 *>(qs + (i * nck + c0 + u) * 4);
                            s[i] = fmaf(qv.x, kv[u].x, s[i]);
                            s[i] = fmaf(qv.y, kv[u].y, s[i]);
                            s[i] = fmaf(qv.z, kv[u].z, s[i]);
                            s[i] = fmaf(qv.w, kv[u].w, s[i]);
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
            gptr vt = as_global(v_cell_ptr(st, bh, slot0)) + (size_t)((slot0 & (PAGE - 1)) >> 6) * ((size_t)TILE * st.Dv * 4);
#pragma unroll 4
            for (int tc = 0; tc < 16; ++tc) {
                kv_f4 vv[NC];
#pragma unroll
                for (int c = 0; c < NC; ++c) {
                    const int col = lane + 64 * c;
                    vv[c] = col < st.Dv ? ld_global<kv_f4>(vt + ((size_t)tc * st.Dv + col) * 16) : kv_f4{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int i = 0; i < RB; ++i) {
                    const kv_f4 pv = *reinterpret_cast<const kv_f4 *>(pw + i * 64 + tc * 4);
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        acc[i][c] = fmaf(pv.x, vv[c].x, acc[i][c]);
                        acc[i][c] = fmaf(pv.y, vv[c].y, acc[i][c]);
                        acc[i][c] = fmaf(pv.z, vv[c].z, acc[i][c]);
                        acc[i][c] = fmaf(pv.w, vv[c].w, acc[i][c]);
                    }
                }
            }
        }
        __syncthreads();
    }

    // ---- the four wavefronts' states into one ------------------------------------------------------
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        float l = lsum[i];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) l += __shfl_xor(l, off);
        if (lane == 0) {
            wml[(wave * RB + i) * 2] = m[i];
            wml[(wave * RB + i) * 2 + 1] = l;
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) wacc[((wave * RB + i) * NC + c) * 64 + lane] = acc[i][c];
    }
    __syncthreads();
    for (int idx = tid; idx < RB * 64 * NC; idx += FT) {
        const int i = idx / (64 * NC), col = idx % (64 * NC), rr = row0 + i;
        if (rr >= R || col >= st.Dv) continue;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < FW; ++w) M = fmaxf(M, wml[(w * RB + i) * 2]);
        float Lt = 0.f, A = 0.f;
#pragma unroll
        for (int w = 0; w < FW; ++w) {
            const float mw = wml[(w * RB + i) * 2];
            const float f = mw > -INFINITY ? expf(mw - M) : 0.f;
            Lt += wml[(w * RB + i) * 2 + 1] * f;
            A += wacc[((w * RB + i) * NC + (col >> 6)) * 64 + (col & 63)] * f;
        }
        if (nparts == 1) {
            const int hq = h * r + rr / a.L, l = rr % a.L;
            reinterpret_cast<float *>(a.out)[((size_t)(b * a.Hq + hq) * a.L + l) * st.Dv + col] = Lt > 0.f ? A / Lt : 0.f;
        } else {
            float *dst = a.workspace + ((size_t)(bh * nparts + part) * R + rr) * (st.Dv + 2);
            dst[col] = A;
            if (col == 0) {
                dst[st.Dv] = M;
                dst[st.Dv + 1] = Lt;
            }
        }
    }
}

// grid (R, BH), one wavefront: the partials [bh][part][row][Dv + 2] of one query row into its output row (up to 64 parts:
// lane p weighs part p, then every lane sums its columns over the parts with independent loads)
__global__ void __launch_bounds__(64)
merge_f32_kernel(AttendArgs a, int nparts) {
    __shared__ float ws[64];
    const int rr = blockIdx.x, bh = blockIdx.y, lane = threadIdx.x;
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
    ws[lane] = w;
    __syncthreads();
    const int hq = h * r + rr / a.L, l = rr % a.L;
    float *out = reinterpret_cast<float *>(a.out) + ((size_t)(b * a.Hq + hq) * a.L + l) * Dv;
    for (int col = lane; col < Dv; col += 64) {
        float A = 0.f;
#pragma unroll 8
        for (int p = 0; p < nparts; ++p) A = fmaf(src[p * pitch + col], ws[p], A);
        out[col] = Lt > 0.f ? A / Lt : 0.f;
    }
}

struct PlanF32 {
    int rb, row_blocks, tiles_total, tiles_per_part, nparts;
};

PlanF32 plan_f32(const AttendArgs &a) {
    PlanF32 p;
    const int R = (a.Hq / a.Hkv) * a.L;
    // (16 rows per workgroup would read the keys half as often, but that instance holds one wavefront per SIMD
    // and waits on its scalar loads: measured at 60 % of the 8-row one's rate on prompt chunks)
    p.rb = R <= 4 ? 4 : 8;
    p.row_blocks = (R + p.rb - 1) / p.rb;
    p.tiles_total = (a.slots + TILE - 1) / TILE;
    // enough workgroups for two per CU; a part keeps at least two tiles per wavefront (with one, a single
    // sequence's step over 8192 keys takes 61 us instead of 51)
    const long wgs = (long)p.row_blocks * a.st.BH;
    int n = (int)std::max(1L, std::min<long>(512 / std::max(1L, wgs), p.tiles_total / (2 * FW)));
    n = std::min(n, 64);
    const size_t per_part = (size_t)a.st.BH * R * (a.st.Dv + 2) * sizeof(float);
    if (a.workspace_cap)
        while (n > 1 && per_part * n > a.workspace_cap) --n;
    p.tiles_per_part = (p.tiles_total + n - 1) / n;
    p.nparts = (p.tiles_total + p.tiles_per_part - 1) / p.tiles_per_part;
    return p;
}

}  // namespace

bool attend_f32_supported(const AttendArgs &a) {
    const Store &s = a.st;
    return s.bits == 0 && s.dtype == KVHIP_F32 && s.Dk <= 512 && s.Dv <= 256 && s.BH <= 65535;
}

size_t attend_f32_workspace(const AttendArgs &a) {
    const PlanF32 p = plan_f32(a);
    return p.nparts == 1 ? 0 : (size_t)a.st.BH * p.nparts * (a.Hq / a.Hkv) * a.L * (a.st.Dv + 2) * sizeof(float);
}

hipError_t launch_attend_f32(const AttendArgs &a, hipStream_t s) {
    const PlanF32 p = plan_f32(a);
    const int nc = a.st.Dv <= 64 ? 1 : a.st.Dv <= 128 ? 2 : 4;
    const int nck = (a.st.Dk + 3) / 4;
    const dim3 grid(p.row_blocks, a.st.BH, p.nparts), block(FT);
    const bool sq = a.st.Dk % 4 == 0;
    const size_t lds = ((sq ? 0 : (size_t)p.rb * nck * 4) + (size_t)FW * p.rb * 64 + (size_t)FW * p.rb * 64 * nc + (size_t)FW * p.rb * 2) * sizeof(float);
#define F32(RB, NC)                                                                                                                       \
    do {                                                                                                                                  \
        if (sq) hipLaunchKernelGGL((attend_f32_kernel<RB, NC, true>), grid, block, lds, s, a, p.tiles_total, p.tiles_per_part, p.nparts); \
        else hipLaunchKernelGGL((attend_f32_kernel<RB, NC, false>), grid, block, lds, s, a, p.tiles_total, p.tiles_per_part, p.nparts);   \
    } while (0)
#define F32_NC(RB)                    \
    do {                              \
        if (nc == 1) F32(RB, 1);      \
        else if (nc == 2) F32(RB, 2); \
        else F32(RB, 4);              \
    } while (0)
    profile_mark(s, true);
    if (p.rb == 4) F32_NC(4);
    else F32_NC(8);
    profile_mark(s, false);
#undef F32_NC
#undef F32
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || p.nparts == 1) return e;
    hipLaunchKernelGGL(merge_f32_kernel, dim3((a.Hq / a.Hkv) * a.L, a.st.BH), dim3(64), 0, s, a, p.nparts);
    return hipGetLastError();
}

}  // namespace kvhip
