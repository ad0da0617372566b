// Shared definitions of libkvhip: the device-resident page layout, the
// row-to-slot run table kernels receive, and the kernel launcher prototypes.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "kvhip.h"

namespace kvhip {

// ---------------------------------------------------------------------------
// Page layout
//
// Cached rows live in fixed pages of PAGE tokens.  A page holds, for each plane (K data,
// V data and, for quantized caches, K and V scale/bias pairs), one cell per (batch row,
// kv head): [b*Hkv + h][PAGE rows].  Pages are found through a page table in device
// memory (one PageEntry per page: the address of the page's cells in each plane), so
// they need not be contiguous: growing a cache allocates further pages and appends
// their entries; nothing already written moves or is copied.
//
//  K plane   one row per token in the reference's own order: Dk elements (full
//            precision) or Dk*bits/32 packed uint32 words in MLX's bit order.  A
//            wavefront lane that owns one token reads its whole row as vectors.
//  V plane   transposed per tile of TILE = 64 tokens, so that the PV contraction
//            reads, for one head-dim column, the values of consecutive tokens as
//            one vector: a page cell is [tile 0..3][d 0..Dv-1][64 tokens].
//              full precision  64 elements, token t at index t
//              8 bit   16 words; word t >> 2 holds tokens 4q..4q+3 at byte
//                      positions {0, 2, 1, 3}
//              4 bit   8 words; word t >> 3 holds an octet of tokens at nibble
//                      positions {0, 4, 1, 5, 2, 6, 3, 7}
//              2 bit   4 words; word t >> 4, token t & 15 at bits [2(t&15), +2)
//            The 4/8-bit positions are the order in which a masked word splits into
//            fp16 operand pairs (see kvhip_attend_decode.hip).
//  sb planes per row and group one (scale, bias) pair of the cache dtype.
// ---------------------------------------------------------------------------
constexpr int PAGE = 256;
constexpr int PAGE_SHIFT = 8;
constexpr int TILE = 64;       // tokens per V tile; 4 tiles per page
constexpr int MAXRUNS = 8;

// Where page p keeps its [BH] cells of each plane (ksb / vsb: quantized caches only).
// (K and its pairs are adjacent, V and its pairs likewise: a kernel fetches each half with one load.)
struct PageEntry {
    char *k = nullptr;
    char *ksb = nullptr;
    char *v = nullptr;
    char *vsb = nullptr;
};

struct Store {
    const PageEntry *pt = nullptr;  // page table (device memory), indexed by slot >> PAGE_SHIFT
    int32_t BH = 0;       // B * Hkv
    int32_t Dk = 0, Dv = 0;
    int32_t dtype = 0;    // kvhip_dtype of cached values / of scales and biases
    int32_t es = 2;       // bytes per element of dtype
    int32_t bits = 0;     // 0: full precision
    int32_t gs = 0;
    // bytes one (page, bh) cell occupies in each plane
    uint32_t k_cell = 0, v_cell = 0, ksb_cell = 0, vsb_cell = 0;
    uint32_t k_row = 0;   // bytes per K row
    uint32_t ksb_row = 0, vsb_row = 0;
};

// Contiguous pieces of the presented order: rows [row0, row0+len) live in
// physical slots [phys0, phys0+len).
struct Runs {
    int32_t n = 0;
    int32_t row0[MAXRUNS];
    int32_t phys0[MAXRUNS];
    int32_t len[MAXRUNS];
};

struct MaskDev {
    int32_t mode = 0;   // kvhip_mask_mode
    int32_t dtype = 0;
    const void *data = nullptr;
    int64_t sb = 0, sh = 0, sl = 0;
    int32_t offset = 0, window = 0;
    const int32_t *lengths = nullptr;
    const int32_t *left_pad = nullptr;
};

#if defined(__HIPCC__)
// ---- device-side address helpers -------------------------------------------
// A wave-uniform slot makes the table lookup a scalar load.
__device__ __forceinline__ const char *k_row_ptr(const Store &st, int bh, int slot) {
    return st.pt[slot >> PAGE_SHIFT].k + (size_t)bh * st.k_cell + (size_t)(slot & (PAGE - 1)) * st.k_row;
}
__device__ __forceinline__ const char *ksb_row_ptr(const Store &st, int bh, int slot) {
    return st.pt[slot >> PAGE_SHIFT].ksb + (size_t)bh * st.ksb_cell + (size_t)(slot & (PAGE - 1)) * st.ksb_row;
}
__device__ __forceinline__ const char *vsb_row_ptr(const Store &st, int bh, int slot) {
    return st.pt[slot >> PAGE_SHIFT].vsb + (size_t)bh * st.vsb_cell + (size_t)(slot & (PAGE - 1)) * st.vsb_row;
}
__device__ __forceinline__ const char *v_cell_ptr(const Store &st, int bh, int slot) {
    return st.pt[slot >> PAGE_SHIFT].v + (size_t)bh * st.v_cell;
}
// Full-precision pages are interleaved in 16-byte chunks inside every 64-token tile, so that a
// wavefront whose lanes are the 64 tokens (K) or 64 adjacent columns (V) reads 1 KB contiguous
// per load and is the only load to touch those cache lines:
//   K tile: [chunk of 16/es elements][token 0..63][16 bytes]
//   V tile: [chunk of 16/es tokens][column 0..Dv-1][16 bytes]
// byte offset of element (slot, d) inside its (page, pair) cell:
__device__ __forceinline__ size_t kfp_off(const Store &st, int slot, int d) {
    const int t = slot & (PAGE - 1), epc = 16 / st.es;
    return (size_t)(t >> 6) * ((size_t)TILE * st.k_row) + ((size_t)(d / epc) * TILE + (t & 63)) * 16 + (size_t)(d % epc) * st.es;
}
__device__ __forceinline__ size_t vfp_off(const Store &st, int slot, int d) {
    const int t = slot & (PAGE - 1), epc = 16 / st.es, tk = t & 63;
    return (size_t)(t >> 6) * ((size_t)TILE * st.Dv * st.es) + ((size_t)(tk / epc) * st.Dv + d) * 16 + (size_t)(tk % epc) * st.es;
}
__device__ __forceinline__ const char *k_cell_ptr(const Store &st, int bh, int slot) {
    return st.pt[slot >> PAGE_SHIFT].k + (size_t)bh * st.k_cell;
}
// A pointer taken from the page table is a plain `char *` to the compiler, which then emits FLAT loads
// for it: those count on both the vector-memory and the LDS/scalar counter, and since they may
// complete through either path a wait for one of them has to be a wait for all -- a tile's loads can
// no longer stay in flight behind the previous tile's.  `gptr` states that the memory is device
// memory (address space 1): the loads become GLOBAL loads with counted, in-order waits.
typedef uint32_t kv_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t kv_u2 __attribute__((ext_vector_type(2)));
#define KV_GLOBAL __attribute__((address_space(1)))
typedef const KV_GLOBAL char *gptr;
__device__ __forceinline__ gptr as_global(const void *p) { return (gptr) reinterpret_cast<const char *>(p); }
template <class T> __device__ __forceinline__ T ld_global(gptr p) { return *reinterpret_cast<const KV_GLOBAL T *>(p); }
template <class T> __device__ __forceinline__ T ld_global(gptr p, int i) { return reinterpret_cast<const KV_GLOBAL T *>(p)[i]; }
// The page-table entry of the page that holds a wave-uniform `slot`, fetched again only when the
// page changes: a kernel that walks the slots in tiles smaller than a page keeps the entry in
// scalar registers across the tiles of one page.
__device__ __forceinline__ char *wave_uniform(char *p) {  // tells the compiler: keep it in scalar registers
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<char *>(((uint64_t)hi << 32) | lo);
}
struct PageCursor {
    int page;
    PageEntry e;
    __device__ __forceinline__ void fetch(const Store &st, int p) {
        page = p;
        const PageEntry &src = st.pt[p];
        e.k = wave_uniform(src.k);
        e.ksb = wave_uniform(src.ksb);
        e.v = wave_uniform(src.v);
        e.vsb = wave_uniform(src.vsb);
    }
    // starts on the page of `slot` (any slot the kernel may read: the entry is valid from the start)
    __device__ __forceinline__ PageCursor(const Store &st, int slot) { fetch(st, __builtin_amdgcn_readfirstlane(slot >> PAGE_SHIFT)); }
    __device__ __forceinline__ const PageEntry &at(const Store &st, int slot) {
        const int p = __builtin_amdgcn_readfirstlane(slot >> PAGE_SHIFT);
        if (p != page) fetch(st, p);
        return e;
    }
};
// bit position of token t (0..63 inside its tile) within the V tile row of a column
template <int BITS> __device__ __forceinline__ int v_bitpos(int t) {
    if (BITS == 4) return 32 * (t >> 3) + 4 * (((t & 7) >> 1) + 4 * (t & 1));
    if (BITS == 8) return 32 * (t >> 2) + 8 * (((t & 3) >> 1) + 2 * (t & 1));
    return BITS * t;  // 2 bits, and the widths that do not divide 32 (3, 5, 6): a plain bit stream over the tile
}
// Packed codes are a little-endian bit stream: code j of a row occupies bits [j BITS, (j + 1) BITS) of the row's
// words.  For 2, 4 and 8 bits that is "element k of a 32-bit word at bits [k BITS, (k + 1) BITS)"; for 3, 5 and 6
// bits it is MLX's 8 / 8 / 4 codes in 3 / 5 / 3 bytes, low code first, where a code may straddle two words.
template <int BITS> __device__ __forceinline__ uint32_t stream_code(const uint32_t *w, int j) {
    const int bit = j * BITS, sh = bit & 31;
    uint32_t v = w[bit >> 5] >> sh;
    if ((32 % BITS) != 0 && sh + BITS > 32) v |= w[(bit >> 5) + 1] << (32 - sh);
    return v & ((1u << BITS) - 1u);
}
// the bits that a value `c` placed at bit `pos` of a stream contributes to word `w` of it
__device__ __forceinline__ uint32_t stream_bits(uint32_t c, int pos, int w) {
    const int rel = pos - 32 * w;
    return rel >= 0 ? (rel < 32 ? (c << rel) : 0u) : (c >> -rel);
}
// (quantized pages) byte offset, inside the page cell, of the V tile row (tile of `slot`, column d)
__device__ __forceinline__ size_t v_row_off(const Store &st, int slot, int d) {
    const size_t row_bytes = st.bits ? (size_t)TILE * st.bits / 8 : (size_t)TILE * st.es;
    return ((size_t)((slot & (PAGE - 1)) >> 6) * st.Dv + d) * row_bytes;
}
template <int BITS> __device__ __forceinline__ uint32_t v_code_load(const char *vrow, int t) {
    if ((32 % BITS) != 0) return stream_code<BITS>(reinterpret_cast<const uint32_t *>(vrow), t);
    const int bp = v_bitpos<BITS>(t);
    return (reinterpret_cast<const uint32_t *>(vrow)[bp >> 5] >> (bp & 31)) & ((1u << BITS) - 1u);
}
// presented row of a physical slot, or -1
__device__ __forceinline__ int slot_to_row(const Runs &r, int slot) {
    int row = -1;
#pragma unroll
    for (int i = 0; i < MAXRUNS; ++i) {
        if (i < r.n) {
            const int d = slot - r.phys0[i];
            if (d >= 0 && d < r.len[i]) row = r.row0[i] + d;
        }
    }
    return row;
}
__device__ __forceinline__ int row_to_slot(const Runs &r, int row) {
    int slot = -1;
#pragma unroll
    for (int i = 0; i < MAXRUNS; ++i) {
        if (i < r.n) {
            const int d = row - r.row0[i];
            if (d >= 0 && d < r.len[i]) slot = r.phys0[i] + d;
        }
    }
    return slot;
}
#endif

// Rotary position embedding applied to rows on their way into a kernel: row l of a
// [B, H, L, D] array sits at position pos0 + l (or batch_pos[b] + l).
struct RopeDev {
    int32_t dims = 0;          // leading head-dim elements that rotate (even); 0 = off
    int32_t traditional = 0;   // 1: pairs (2i, 2i+1); 0: pairs (i, i + dims/2)
    float scale = 1.f;         // position scale
    double log_base_over_half = 0.;  // log(base) / (dims/2): pair i turns by position * exp(-i * this)
    const float *freqs = nullptr;    // optional [dims/2]: pair i turns by position / freqs[i]
    int32_t pos0 = 0;
    const int32_t *batch_pos = nullptr;  // optional [B] (device)
    int32_t H = 1;             // heads per batch row of the array being rotated
};

// ---- kernel launchers (defined in the .hip files) ---------------------------
// New rows src[l] for l in [src0, src0+n) go to physical slots [slot0, slot0+n); with `rope`
// the K rows are rotated (and rounded to the cache dtype) on the way in.
hipError_t launch_append_fp(const Store &st, const void *keys, const void *values, int L, int src0,
                            int slot0, int n, hipStream_t s, const RopeDev *rope = nullptr);
hipError_t launch_append_quant(const Store &st, const void *keys, const void *values, int L, int src0,
                               int slot0, int n, hipStream_t s, const RopeDev *rope = nullptr);
// out = rope(x) for x [B, H, L, D] of `dtype` (out may alias x)
hipError_t launch_rope_apply(const RopeDev &rope, const void *x, void *out, int B, int H, int L, int D,
                             int dtype, hipStream_t s);
// Copy rows [row_begin, row_begin+count) of `runs` out to dense [BH, dst_rows, D] arrays whose
// row 0 corresponds to row dst_row0 of `runs`.  Either destination may be NULL.
hipError_t launch_export_fp(const Store &st, const Runs &runs, int row_begin, int count, int dst_row0,
                            int dst_rows, void *dst_k, void *dst_v, hipStream_t s);
// which: 0 k.wq 1 k.scales 2 k.biases 3 v.wq 4 v.scales 5 v.biases
hipError_t launch_export_quant(const Store &st, int which, int nrows, void *dst, hipStream_t s);
// Dense [BH, nrows, D] arrays into slots [0, nrows).
hipError_t launch_import_fp(const Store &st, const void *src_k, const void *src_v, int nrows, hipStream_t s);
hipError_t launch_import_quant(const Store &st, const void *const srcs[6], int nrows, hipStream_t s);
// Device-to-device copy of slots between two stores of identical geometry, through a row map:
// dst slot i <- src slot of presented row i.
hipError_t launch_compact_fp(const Store &src, const Runs &runs, const Store &dst, int nrows, hipStream_t s);
// Rows [0, rows) of the full-precision store `src` quantized into the same slots of `dst`
// (`KVCacheSimple.toQuantized`), and the reverse (`QuantizedKVCache.toUnquantized`): one pass
// from pages to pages, no dense copy in between.
hipError_t launch_requant_pages(const Store &src, const Store &dst, int rows, hipStream_t s);
hipError_t launch_dequant_pages(const Store &q, const Store &dst, int rows, hipStream_t s);
hipError_t launch_dequant_scratch(const Store &q, const Store &dst, int rows, int pages, const PageEntry &page0, size_t sk, size_t sv,
                                  hipStream_t s);
// The whole-tile quantizer for 2-, 3-, 5- and 6-bit codes (kvhip_quant_tile_other.hip): `tiles` tiles of dense rows
// from row a0 on into the slots from b0 on, and tiles [0, tiles) of a full-precision page store into the same slots.
hipError_t launch_quant_tiles_other(const Store &st, const void *keys, const void *values, int L, int a0, int b0, int tiles,
                                    hipStream_t s, const RopeDev &r);
hipError_t launch_requant_tiles_other(const Store &src, const Store &st, int tiles, hipStream_t s);
hipError_t launch_affine_quantize(const void *src, int64_t rows, int D, int gs, int bits, int dtype,
                                  uint32_t *wq, void *scales, void *biases, hipStream_t s);
hipError_t launch_affine_dequantize(const uint32_t *wq, const void *scales, const void *biases,
                                    int64_t rows, int D, int gs, int bits, int dtype, void *dst,
                                    hipStream_t s);
hipError_t launch_mask_materialize(const kvhip_mask_plan_t &plan, uint8_t *dst, hipStream_t s);
// Zero / copy `bytes` of device memory with a kernel (16-byte aligned pointers and sizes).
hipError_t launch_fill_zero(void *dst, size_t bytes, hipStream_t s);
hipError_t launch_copy_bytes(void *dst, const void *src, size_t bytes, hipStream_t s);
// `rows` dense rows of src_pitch bytes into rows of dst_pitch bytes (both even): common prefix copied, rest zero-filled
hipError_t launch_repitch_rows(void *dst, size_t dst_pitch, const void *src, size_t src_pitch, size_t rows, hipStream_t s);
// Page-table entries [first, first + count): page first + i keeps its cells at base.x + i * stride.x
// for each plane x (pages backed by one allocation lie at a regular stride).
hipError_t launch_set_pages(PageEntry *pt, int first, int count, PageEntry base, const size_t stride[4], hipStream_t s);
// Every plane of pages [0, pages) of `src` into the same pages of `dst` (stores of one geometry).
hipError_t launch_copy_pages(const Store &src, const Store &dst, int pages, hipStream_t s);

struct AttendArgs {
    Store st;
    Runs runs;
    const void *q = nullptr;  // [B, Hq, L, Dk]
    void *out = nullptr;      // [B, Hq, L, Dv]
    int32_t B = 0, Hq = 0, Hkv = 0, L = 0;
    int32_t T = 0;            // presented length
    int32_t slots = 0;        // physical slots in use span [0, slots)
    float scale = 1.f;
    MaskDev mask;
    float *workspace = nullptr;
    size_t workspace_bytes = 0;
    // Single-token decode (`attentionWithCacheUpdate` with L = 1): the new row [BH, 1, D] of keys and
    // values, still to be written (quantized caches: quantized) into physical slot `new_slot`.  The decode
    // kernel does it itself -- the wavefront that reads the slot's tile writes the row first -- so a
    // step needs no launch for the append.  NULL: the row is already in the cache.
    const void *new_k = nullptr;
    const void *new_v = nullptr;
    int new_slot = -1;
    // Upper bound on the scratch a launch may plan for (0: none).  The planners then split the sequence over
    // fewer spans or key-range parts, down to one, which needs no scratch at all.
    size_t workspace_cap = 0;
};
// Whether launch_attend_decode writes a.new_k / a.new_v itself for these arguments.
bool attend_decode_fuses_append(const AttendArgs &a);
// Bytes of scratch each kernel family needs for these arguments.
size_t attend_generic_workspace(const AttendArgs &a);
hipError_t launch_attend_generic(const AttendArgs &a, hipStream_t s);
// Full-precision caches on the vector ALUs (float32 caches; 16-bit ones of head sizes above 256, which the matrix-core
// kernels are not built for; keys up to 1024 wide, values up to 512): any row count, any mask.
bool attend_valu_supported(const AttendArgs &a);
// Whether a quantized cache none of the quantized kernels take (head sizes above 256) can be dequantized into scratch
// pages for this kernel.
bool attend_valu_dequant_first(const AttendArgs &a);
size_t attend_valu_workspace(const AttendArgs &a);
hipError_t launch_attend_valu(const AttendArgs &a, hipStream_t s);
// Fast split-sequence decode kernels; `supported` says whether the shape is covered.
bool attend_decode_supported(const AttendArgs &a);
size_t attend_decode_workspace(const AttendArgs &a);
hipError_t launch_attend_decode(const AttendArgs &a, hipStream_t s);
// Matrix-core chunked-prefill tile (many query rows per kv head).
bool attend_prefill_supported(const AttendArgs &a);
size_t attend_prefill_workspace(const AttendArgs &a);
// Whether a prompt chunk over a quantized cache is faster with the cache dequantized into scratch pages first and the
// full-precision tile run over them (many query rows per kv head share the one conversion of every cached row).
// (`always`: whenever the shape allows it, whatever the row count)
bool attend_prefill_dequant_first(const AttendArgs &a, bool always);
// After the full-precision tile has run over a dequantized copy of a quantized cache: query rows whose mask excludes
// every key take the reference's quantized answer, equal weights over all T keys (a.st: the dequantized pages).
// `mask_may_...`: false when the mask provably leaves no such row, so the launch can be left out.
bool mask_may_leave_rows_without_keys(const AttendArgs &a);
hipError_t launch_rows_without_keys(const AttendArgs &a, hipStream_t s);
// Merge `nsplit` partials per query row, laid out [bh][split][rows][D+2] in a.workspace
// (out[D] unnormalised, running max, running sum), and write the normalised rows to a.out.
hipError_t launch_combine(const AttendArgs &a, int nsplit, int rows, hipStream_t s);
hipError_t launch_attend_prefill(const AttendArgs &a, hipStream_t s);
hipError_t launch_attend_decode16(const AttendArgs &a, int tiles_total, int tiles_per_wg, int nsplit, hipStream_t s);
// (2- / 3-bit and 5- / 6-bit instances of the same kernel, and the shapes they are built for)
hipError_t launch_attend_decode16_low(const AttendArgs &a, int tiles_total, int tiles_per_wg, int nsplit, hipStream_t s);
hipError_t launch_attend_decode16_high(const AttendArgs &a, int tiles_total, int tiles_per_wg, int nsplit, hipStream_t s);
bool decode16_stream_shape(const Store &s);
hipError_t launch_attend_prefill_fp(const AttendArgs &a, int nsplit, bool wide, hipStream_t s);
// The pipelined tile for quantized caches (head sizes 64 / 128 / 256, slots in presented order).
bool attend_prefill_q_supported(const AttendArgs &a);
// rows: query rows per workgroup, 64 (4 wavefronts) or 256 (8 wavefronts; head size 128)
hipError_t launch_attend_prefill_q(const AttendArgs &a, int nsplit, int rows, hipStream_t s);
hipError_t launch_attend_prefill_q_other(const AttendArgs &a, int nsplit, int rows, hipStream_t s);  // 2-, 3-, 5- and 6-bit codes
// Switches for timing experiments (forced span sizes and the like) are read from the environment only in a
// library built with -DKVHIP_MEASURE; the shipped build compiles every one of them to its default.
#ifdef KVHIP_MEASURE
inline int measure_knob(const char *name, int dflt) {
    const char *v = getenv(name);
    return v ? atoi(v) : dflt;
}
#else
constexpr int measure_knob(const char *, int dflt) { return dflt; }
#endif
// Event bracket around the dominant kernel while profiling is enabled.
void profile_enable(int every);
void profile_mark(hipStream_t s, bool begin);
hipError_t profile_read(int *launches, double *total_ms);

}  // namespace kvhip
