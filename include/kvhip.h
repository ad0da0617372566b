/*
 * kvhip.h -- C interface of libkvhip.so, the MI355X (gfx950) implementation of
 * the KV-cache hot path of mlx-swift-lm.
 *
 * A Swift system-library target imports this header (and nothing else) through
 * a module map, in the way Libraries/MLXCXGrammar/include/module.modulemap
 * exposes xgrammar_c.h.  One `kvhip_cache` handle stands behind one instance of
 * the reference's `KVCacheSimple`, `RotatingKVCache` or `QuantizedKVCache`
 * (Libraries/MLXLMCommon/KVCache.swift:391, :541, :923); every entry point
 * below names the reference member it replaces.
 *
 * Conventions
 *  - Every pointer named `keys`, `values`, `queries`, `out`, `dst`, `src` or
 *    `data` is a DEVICE pointer to a dense row-major array; shapes are given in
 *    the comment of each function.  Inputs are borrowed for the duration of the
 *    call's enqueued work only.  The element type's own alignment suffices (a
 *    contiguous view that starts anywhere inside an allocation is accepted);
 *    16-byte aligned arrays are read at full width.
 *  - `stream` is a `hipStream_t` passed as `void *` (NULL = the default
 *    stream).  Device work is enqueued on it; host-side counters (`offset`,
 *    `idx`) advance when the call returns, as the reference's do while it
 *    builds its lazy graph (KVCache.swift:438, :729-730, :1067).
 *  - A handle is not thread-safe: like the reference's `KVCacheStorage`
 *    (KVCachePlan.swift:104-111) it is externally serialised by its owner.
 *  - Fallible functions return a status: 0 on success, negative on failure,
 *    with a message readable through kvhip_last_error_message() on the calling
 *    thread (idiom of xgrammar_c.h:39-69).
 */
#ifndef KVHIP_H
#define KVHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t kvhip_status;
#define KVHIP_OK               ((int32_t)0)
#define KVHIP_ERR_INTERNAL     ((int32_t)-1)
#define KVHIP_ERR_INVALID_ARG  ((int32_t)-2)
#define KVHIP_ERR_UNSUPPORTED  ((int32_t)-3) /* shape / dtype / bit width outside what the kernels cover */
#define KVHIP_ERR_STATE        ((int32_t)-4) /* a call the reference answers with fatalError / throws */
#define KVHIP_ERR_HIP          ((int32_t)-5) /* a HIP runtime call failed */
#define KVHIP_ERR_NO_DEVICE    ((int32_t)-6) /* no gfx950 device visible */

typedef enum {
    KVHIP_KIND_SIMPLE = 0,    /* KVCacheSimple    KVCache.swift:391-538  */
    KVHIP_KIND_ROTATING = 1,  /* RotatingKVCache  KVCache.swift:541-900  */
    KVHIP_KIND_QUANTIZED = 2, /* QuantizedKVCache KVCache.swift:923-1210 */
} kvhip_kind;

typedef enum {
    KVHIP_F16 = 0,
    KVHIP_BF16 = 1,
    KVHIP_F32 = 2,
    KVHIP_U32 = 3,  /* packed codes in exported state */
    KVHIP_BOOL = 4, /* one byte per element, for masks */
} kvhip_dtype;

/* Constructor arguments of the three cache classes.  Fields a kind does not
 * use are ignored.  step <= 0 selects the reference default (256). */
typedef struct {
    int32_t kind;       /* kvhip_kind */
    int32_t step;       /* KVCacheSimple.step :394, RotatingKVCache(step:) :565 */
    int32_t max_size;   /* RotatingKVCache(maxSize:) */
    int32_t keep;       /* RotatingKVCache(keep:) */
    int32_t group_size; /* QuantizedKVCache(groupSize:) :931 */
    int32_t bits;       /* QuantizedKVCache(bits:), affine mode; 2, 3, 4, 5, 6 or 8 */
} kvhip_config;

/* MLXFast.ScaledDotProductAttentionMaskMode as the attention entry points take it. */
typedef enum {
    KVHIP_MASK_NONE = 0,
    KVHIP_MASK_CAUSAL = 1, /* query i sees key j iff j <= T - L + i (KVCache.swift:2396-2400) */
    KVHIP_MASK_ARRAY = 2,  /* bool: keep where true; float: added to the scores (:2436-2446) */
    /* createCausalMask(n:, offset:, windowSize:, lengths:) (KVCache.swift:253-275)
     * evaluated from indices inside the kernel instead of being materialised:
     * keep iff offset+i >= j && (window <= 0 || offset+i < j + window)
     *       && (lengths == NULL || j < lengths[b]) && (left_pad == NULL || j >= left_pad[b]) */
    KVHIP_MASK_WINDOW = 3,
} kvhip_mask_mode;

typedef struct {
    int32_t mode;       /* kvhip_mask_mode */
    int32_t dtype;      /* ARRAY: KVHIP_BOOL, KVHIP_F16, KVHIP_BF16 or KVHIP_F32 */
    const void *data;   /* ARRAY: device pointer, innermost (key) axis contiguous */
    int64_t stride_b;   /* ARRAY: element strides of the batch, query-head and query-row */
    int64_t stride_h;   /*        axes; 0 broadcasts the axis                            */
    int64_t stride_l;
    int32_t key_len;    /* ARRAY: extent of the key axis (must equal the presented length) */
    int32_t offset;     /* WINDOW */
    int32_t window;     /* WINDOW: <= 0 means no window */
    const int32_t *lengths;  /* WINDOW: optional device [B] */
    const int32_t *left_pad; /* WINDOW: optional device [B] */
} kvhip_mask;

/* What `makeMask(n:windowSize:returnArray:)` decides (KVCache.swift:236-250,
 * :834-871): a symbolic mode, or the parameters of the array it would build. */
typedef struct {
    int32_t mode;      /* NONE, CAUSAL, or ARRAY (the reference would materialise an array) */
    int32_t rows;      /* ARRAY: n */
    int32_t cols;      /* ARRAY: key extent */
    int32_t offset;    /* ARRAY from createCausalMask: its `offset` argument */
    int32_t window;    /* ARRAY from createCausalMask: windowSize, or 0 */
    int32_t rolled;    /* 1: the single-token rolled window mask of RotatingKVCache.makeMask :855-868 */
    int32_t roll_shift;/* rolled: currentIdx + 1 */
    int32_t roll_window;
} kvhip_mask_plan_t;

typedef struct kvhip_cache kvhip_cache;

/* ---- library ----------------------------------------------------------- */
const char *kvhip_version(void);
/* Message of the last failure on this thread, or NULL. Valid until the next kvhip call. */
const char *kvhip_last_error_message(void);
/* Binds the library to HIP device `device` (default 0) and checks it is gfx950. */
kvhip_status kvhip_init(int32_t device);
/* Blocks until all work enqueued on `stream` is done (tests; `eval(cache)` LLMModel.swift:56-58).
 * Also releases device memory of freed caches and replaced buffers whose last readers are done. */
kvhip_status kvhip_sync(void *stream);
/* 0 = choose the fastest kernel for the shape (default); 1 = always the generic kernel; 2 and 3 = as 0, but a
 * prompt chunk over a quantized cache never (2) or whenever the shape allows (3) runs dequantize-first -- the
 * cached rows converted once into scratch pages, then the full-precision tile -- instead of by row count.
 * The setting, kvhip_last_attend_kernel and the profile record below belong to the calling thread. */
void kvhip_set_kernel_policy(int32_t policy);
/*
 * Measurement hooks (no counterpart in the reference, which times whole
 * generations with wall clocks, Evaluate.swift:2467).  kvhip_profile_enable(n) with n > 0
 * brackets every n-th launch of the dominant attention kernel (split-sequence decode or
 * prefill tile) with HIP events on the stream it is launched on (n = 1: every launch; a
 * larger n keeps the event packets, a few microseconds per bracket, out of most steps of a
 * timed loop); 0 switches it off.  kvhip_profile_read waits for those events, returns the
 * number of bracketed launches and their summed duration in milliseconds, and clears the record.
 */
/* Which kernel family the last attention call on this thread's library state used:
 * 0 generic, 1 matrix-core decode (quantized), 2 matrix-core decode (full precision),
 * 3 matrix-core chunked-prefill tile, 4 the same tile over scratch pages a quantized cache was dequantized into
 * first, 5 the vector-ALU kernel (float32 caches, 16-bit head sizes above 256), 6 the same over scratch pages a
 * quantized cache of such head sizes, or one with float32 scales, was dequantized into first; -1 before the first
 * call.  For tests and reports. */
int32_t kvhip_last_attend_kernel(void);
void kvhip_profile_enable(int32_t every);
kvhip_status kvhip_profile_read(int32_t *out_launches, double *out_total_ms);

/* ---- lifetime ---------------------------------------------------------- */
/* KVCacheSimple() / RotatingKVCache(maxSize:keep:step:) / QuantizedKVCache(groupSize:bits:) */
kvhip_status kvhip_cache_create(const kvhip_config *config, kvhip_cache **out_cache);
/* Safe with NULL.  Does not wait for the device: the cache's memory is released once the work
 * enqueued on the stream it was last used with has run (by a later kvhip_sync / kvhip_cache_reserve,
 * or at once if that stream is idle), and is then kept for reuse by later allocations of a similar size.
 * Only the last stream is tracked: a caller that reads one cache from several streams has to order them
 * (an event wait on the last one) before it frees the cache. */
void kvhip_cache_free(kvhip_cache *cache);
/* `copy()` (KVCache.swift:525-533, :877-885, :1177-1185): independent deep copy. */
kvhip_status kvhip_cache_copy(const kvhip_cache *cache, void *stream, kvhip_cache **out_cache);
/* Optional: allocate the device pages for `tokens` cached rows in one piece.  Updates grow a cache by
 * themselves (further pages are allocated and entered into its page table; nothing is copied and the
 * call does not wait for the device), so this only saves those allocations.  It has no stream
 * argument: its zero-fill runs on the default stream and the call waits for it, so that a first
 * update on any stream is ordered after it. */
kvhip_status kvhip_cache_reserve(kvhip_cache *cache, int32_t B, int32_t Hkv, int32_t Dk, int32_t Dv,
                                 int32_t dtype, int64_t tokens);

/* ---- the KVCache protocol surface (KVCache.swift:46-104) ----------------- */
int64_t kvhip_cache_offset(const kvhip_cache *cache);          /* `offset` */
int64_t kvhip_cache_idx(const kvhip_cache *cache);             /* RotatingKVCache.idx (metaState[4]) */
int64_t kvhip_cache_max_size(const kvhip_cache *cache);        /* `maxSize`, -1 for nil */
int32_t kvhip_cache_group_size(const kvhip_cache *cache);      /* QuantizedKVCacheProtocol.groupSize */
int32_t kvhip_cache_bits(const kvhip_cache *cache);            /* QuantizedKVCacheProtocol.bits */
int64_t kvhip_cache_capacity(const kvhip_cache *cache);        /* row extent of the reference's buffers */
int64_t kvhip_cache_presented_length(const kvhip_cache *cache);/* key extent `update` last returned */
/* Rows the device pages allocated so far can hold (a multiple of 256).  No counterpart in the
 * reference, whose `capacity` above is the extent of its arrays; for tests and measurements. */
int64_t kvhip_cache_device_rows(const kvhip_cache *cache);
/* Device slots a decode launch walks: one past the highest slot that holds a presented row.  Equal to
 * the presented length except for a RotatingKVCache whose prompt chunks left unused slots between its
 * rows (they are squeezed out once when the full ring settles into single-token steps).  No counterpart
 * in the reference; for tests and measurements. */
int64_t kvhip_cache_slot_span(const kvhip_cache *cache);
int32_t kvhip_cache_is_trimmable(const kvhip_cache *cache, int64_t after_positions); /* isTrimmable(after:) */
int64_t kvhip_cache_trim(kvhip_cache *cache, int64_t n);       /* trim(_:) -> positions trimmed */
/* `offset` is a settable stored property in the reference (KVCache.swift:185;
 * used by toQuantized :504 and toUnquantized :1190). */
kvhip_status kvhip_cache_set_offset(kvhip_cache *cache, int64_t offset);

/*
 * `update(keys:values:)` (Simple :404-447, Rotating :742-750) and
 * `updateQuantized(keys:values:)` (:1011-1102).
 * keys [B,Hkv,L,Dk], values [B,Hkv,L,Dv] of `dtype`.  Appends / ring-writes /
 * quantizes on the device; advances offset (and idx).  What the reference
 * returns -- every cached row in presentation order -- stays on the device and
 * is read by kvhip_cache_attend, or copied out by kvhip_cache_fetch*.
 */
kvhip_status kvhip_cache_update(kvhip_cache *cache, const void *keys, const void *values, int32_t B,
                                int32_t Hkv, int32_t L, int32_t Dk, int32_t Dv, int32_t dtype,
                                void *stream);

/* ---- rotary positions on the way in ----------------------------------------- */
/*
 * The rotary embedding a model applies to queries and keys immediately before the cache
 * write (`applyRotaryPosition(rope, to:, offset: cache?.ropeOffset)`, Llama.swift:58-60,
 * RoPEApplication.swift:62-74; the layers call `MLXFast.RoPE(x, dimensions:, traditional:,
 * base:, scale:, offset:, freqs:)`, RoPEUtils.swift:139-156, SuScaledRoPE.swift:49-70).
 * The first `dims` elements of each head rotate: pairs (2i, 2i+1) when `traditional`, else
 * (i, i + dims/2); pair i of the row at position p turns by p * scale * base^(-2i/dims), or by
 * p * scale / freqs[i] when `freqs` (a device array of dims/2 floats) is given.  Angles and
 * products are float32, the result is rounded once to the array's dtype.
 */
typedef struct kvhip_rope {
    int32_t dims;
    int32_t traditional;
    float base;
    float scale;
    const float *freqs; /* device, or NULL */
} kvhip_rope;

/* out = rope(x) for x [B,H,L,D]; row l sits at position offset + l, or batch_offsets[b] + l
 * when batch_offsets (device, [B]: `RoPEOffset.batch`, RoPEApplication.swift:13-23) is given.
 * out may be x. */
kvhip_status kvhip_rope_apply(const kvhip_rope *rope, const void *x, void *out, int32_t B, int32_t H,
                              int32_t L, int32_t D, int32_t dtype, int64_t offset,
                              const int32_t *batch_offsets, void *stream);

/* `kvhip_cache_update` with the keys rotated inside the append / quantize-on-append kernel
 * (no rotated copy of the keys is written).  Positions start at the cache's `ropeOffset`:
 * its offset before this write (plus the staged rows of an open round), or batch_offsets[b]. */
kvhip_status kvhip_cache_update_rope(kvhip_cache *cache, const kvhip_rope *rope, const int32_t *batch_offsets,
                                     const void *keys, const void *values, int32_t B, int32_t Hkv,
                                     int32_t L, int32_t Dk, int32_t Dv, int32_t dtype, void *stream);

/* The arrays the last `update` returned: dst_keys [B,Hkv,P,Dk], dst_values
 * [B,Hkv,P,Dv], P = kvhip_cache_presented_length.  Not for quantized caches. */
kvhip_status kvhip_cache_fetch(const kvhip_cache *cache, void *dst_keys, void *dst_values, void *stream);

/*
 * Attention over what the cache presents, replacing
 * `MLXFast.scaledDotProductAttention` (AttentionUtils.swift:86-93) for Simple /
 * Rotating caches and `quantizedScaledDotProductAttention`
 * (KVCache.swift:2351-2447) for quantized ones.
 * queries [B,Hq,L,Dk] and out [B,Hq,L,Dv] in the cache's dtype.
 * Every dtype, bit width, head size, group size and mask is accepted.  The tuned kernels take
 * float16 / bfloat16 caches with Dk == Dv in {64, 96, 128, 256}, keys of 192 with values of 128 (also
 * 80 when not quantized; quantized: every code width, group size 32, 64 or 128).  A 16-bit cache
 * of other head sizes up to 256 stores its rows zero-padded to the next of those sizes (112 as 128,
 * 160 as 256) and runs the same kernels; every array that crosses this interface keeps the caller's
 * head sizes.  float32 caches and 16-bit caches of head sizes above 256 (not quantized; keys up to
 * 1024 wide, values up to 512) run on a vector-ALU kernel, bound by the memory system at a few query
 * rows per kv head and by float32 arithmetic on prompt chunks.  A quantized cache of head sizes above
 * 256, or one with float32 scales, is dequantized into pooled scratch pages at every call and runs the
 * same kernel over them (the allocation-free entry point does not: it uses the plain kernel, which is
 * 50-75 times slower than the tuned ones at 8k keys and otherwise only serves head sizes above 1024 /
 * 512 and kvhip_set_kernel_policy(1)).  kvhip_last_attend_kernel() tells which one ran.
 */
kvhip_status kvhip_cache_attend(kvhip_cache *cache, const void *queries, int32_t B, int32_t Hq,
                                int32_t L, int32_t D, float scale, const kvhip_mask *mask, void *out,
                                void *stream);

/*
 * kvhip_cache_attend for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, same kernels and the same results as kvhip_cache_attend, but the
 * kernels' scratch (the partial results of the sequence spans) lives in a fixed array of
 * KVHIP_STATIC_SCRATCH_BYTES that every device the library was initialised on holds until the
 * process ends, and the call makes no hipMalloc / hipFree.  The tuned kernels plan for that
 * amount: they divide the sequence over fewer spans or key-range parts until the partials fit
 * (a single span or part needs none), so they take every shape; where that gives another number of
 * parts than kvhip_cache_attend would use, the float32 sums are formed in another order; and a large
 * prompt chunk over a quantized cache, which kvhip_cache_attend runs over a dequantized copy in pooled
 * scratch pages, runs on the quantized tile here (the same result within the rounding of intermediates).  Only the
 * plain kernel, which keeps one float per (query row, key), can need more than the array holds: such
 * a call returns KVHIP_ERR_UNSUPPORTED and enqueues nothing.  Nothing in the array has to start from zero:
 * each span writes its partial before the merge reads it.  All calls on one device share the
 * array, so two calls whose device work can overlap (different streams, or a captured graph
 * replayed beside eager calls) race; calls on one stream are ordered and safe.
 * Requires kvhip_init on the current device.
 */
#define KVHIP_STATIC_SCRATCH_BYTES (16u << 20)
kvhip_status kvhip_cache_attend_static(kvhip_cache *cache, const void *queries, int32_t B, int32_t Hq,
                                       int32_t L, int32_t D, float scale, const kvhip_mask *mask,
                                       void *out, void *stream);

/* `attentionWithCacheUpdate` (AttentionUtils.swift:37-95): update, then attend.  A single new token without a
 * mask is written by the decode kernel itself where one of them serves the call (quantized caches up to sixteen
 * query heads per kv head, 16-bit full-precision caches up to eight): the step then has no launch for the append. */
kvhip_status kvhip_cache_update_attend(kvhip_cache *cache, const void *queries, const void *keys,
                                       const void *values, int32_t B, int32_t Hq, int32_t Hkv,
                                       int32_t L, int32_t Dk, int32_t Dv, int32_t dtype, float scale,
                                       const kvhip_mask *mask, void *out, void *stream);

/* `makeMask(n:windowSize:returnArray:)`; window_size <= 0 stands for nil. */
kvhip_status kvhip_cache_mask_plan(const kvhip_cache *cache, int32_t n, int32_t window_size,
                                   int32_t return_array, kvhip_mask_plan_t *out_plan);
/* Writes the bool array the plan describes: dst [rows, cols] (or [cols] when rolled), one byte each. */
kvhip_status kvhip_mask_materialize(const kvhip_mask_plan_t *plan, uint8_t *dst, void *stream);

/* ---- state / metaState (serialisation surface) --------------------------- */
/*
 * `state` getter: Simple/Rotating [keys, values]; Quantized [k.wq, k.scales,
 * k.biases, v.wq, v.scales, v.biases] (KVCache.swift:449-460, :752-763,
 * :1113-1130), each [B,Hkv,rows,last].  Count is 0 before the first write.
 */
int32_t kvhip_cache_state_count(const kvhip_cache *cache);
kvhip_status kvhip_cache_state_desc(const kvhip_cache *cache, int32_t index, int64_t shape[4],
                                    int32_t *dtype);
kvhip_status kvhip_cache_state_export(const kvhip_cache *cache, int32_t index, void *dst, void *stream);
/*
 * `state` setter (KVCache.swift:461-468, :764-773, :1131-1146): `count` arrays in
 * the getter's order, shapes[i] = 4 extents, dtypes[i] a kvhip_dtype.  Simple
 * sets offset to the row extent; Rotating and Quantized leave offset to metaState.
 */
kvhip_status kvhip_cache_state_import(kvhip_cache *cache, int32_t count, const void *const *srcs,
                                      const int64_t *shapes, const int32_t *dtypes, void *stream);
/* `metaState`: Simple [""]; Rotating [keep,maxSize,step,offset,idx,origin];
 * Quantized [step,offset,groupSize,bits] (KVCache.swift:207-214, :775-815, :1148-1166). */
int32_t kvhip_cache_meta_count(const kvhip_cache *cache);
/* Copies entry `index` (NUL-terminated) into buf; returns its length, or a negative status. */
int32_t kvhip_cache_meta_get(const kvhip_cache *cache, int32_t index, char *buf, int32_t buf_len);
kvhip_status kvhip_cache_meta_set(kvhip_cache *cache, int32_t count, const char *const *values);

/* ---- staged rounds on a ring ------------------------------------------------ */
/*
 * `RotatingStagedKVCache` (RotatingStagedKVCache.swift:12-132) and the rotating leaf of a
 * speculative round (`RotatingRoundStrategy`, KVCacheRound.swift:128-156), folded into the
 * ring's own handle.  Between `stage_begin` and `stage_commit` the handle behaves as the
 * staged wrapper:
 *   - `kvhip_cache_update` stages its rows (device copy into spare slots; the ring and its
 *     offset / idx stay untouched) and the presentation becomes
 *     logicalView(tail: min(offset, maxSize-1)) ++ staged (RotatingStagedKVCache.swift:78-91),
 *     which `kvhip_cache_fetch` exports and `kvhip_cache_attend` reads in place;
 *   - offset, idx, is_trimmable, trim, state export, meta_get and `kvhip_cache_mask_plan`
 *     keep answering for the live ring, which does not move (:49-58, :95-111); the
 *     wrapper's own `offset` is kvhip_cache_offset + kvhip_cache_stage_count (:33-37), its
 *     `isTrimmable` is false and its `trim` returns 0 (:113-119) -- the host shim says so
 *     without a call;
 *   - state import, meta_set and copy fail with KVHIP_ERR_STATE (the reference traps).
 * Only KVHIP_KIND_ROTATING stages; the other kinds are written through and trimmed
 * (`AppendOnlyRoundStrategy`, KVCacheRound.swift:99-125) and get KVHIP_ERR_INVALID_ARG here.
 */
kvhip_status kvhip_cache_stage_begin(kvhip_cache *cache);
int32_t kvhip_cache_stage_is_open(const kvhip_cache *cache);
/* `stagedCount` (RotatingStagedKVCache.swift:23). */
int64_t kvhip_cache_stage_count(const kvhip_cache *cache);
/* `stagedArrays` (RotatingStagedKVCache.swift:27-30): the staged rows as [B,Hkv,n,D] pairs. */
kvhip_status kvhip_cache_stage_fetch(const kvhip_cache *cache, void *dst_keys, void *dst_values, void *stream);
/*
 * `commit(retaining:)` (RotatingStagedKVCache.swift:62-76): the first
 * min(max(retaining,0), staged) rows are appended to the ring through the normal write
 * path (`kvhip_cache_update` semantics for that many rows), the rest are dropped, and the
 * round closes.  retaining = 0 is a rollback.
 */
kvhip_status kvhip_cache_stage_commit(kvhip_cache *cache, int64_t retaining, void *stream);

/* ---- ring reads and conversions ------------------------------------------ */
/*
 * `RotatingKVCache.logicalView(tail:)` (KVCache.swift:631-658): chronological
 * trailing entries without mutating the ring.  *out_rows receives
 * n = max(min(max(tail,0),count), min(keep,count)); with non-NULL dst pointers
 * the rows are written as [B,Hkv,n,D].  Returns KVHIP_ERR_STATE before the first write.
 */
kvhip_status kvhip_cache_logical_view(const kvhip_cache *cache, int64_t tail, int64_t *out_rows,
                                      void *dst_keys, void *dst_values, void *stream);
/* `KVCacheSimple.toQuantized(groupSize:bits:)` (KVCache.swift:486-523): one kernel that quantizes
 * from the full-precision pages into the new cache's pages (no dense copy, no wait for the device). */
kvhip_status kvhip_cache_to_quantized(const kvhip_cache *cache, int32_t group_size, int32_t bits,
                                      void *stream, kvhip_cache **out_cache);
/* `QuantizedKVCache.toUnquantized()` (KVCache.swift:1188-1209). */
kvhip_status kvhip_cache_to_unquantized(const kvhip_cache *cache, void *stream, kvhip_cache **out_cache);
/* `resolvedKVQuantizationGroupSize` (KVCache.swift:902-920); 0 when none fits. */
int32_t kvhip_resolved_group_size(int32_t requested, int32_t key_head_dim, int32_t value_head_dim);

/* ---- standalone quantizer (MLX.quantized / MLX.dequantized call sites) ---- */
/* src [rows, D] of `dtype` -> wq [rows, D*bits/32] u32, scales/biases [rows, D/group_size] of `dtype`. */
kvhip_status kvhip_affine_quantize(const void *src, int64_t rows, int32_t D, int32_t group_size,
                                   int32_t bits, int32_t dtype, uint32_t *wq, void *scales,
                                   void *biases, void *stream);
kvhip_status kvhip_affine_dequantize(const uint32_t *wq, const void *scales, const void *biases,
                                     int64_t rows, int32_t D, int32_t group_size, int32_t bits,
                                     int32_t dtype, void *dst, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KVHIP_H */
