// Host side of libkvhip: the three cache state machines of the reference
// (offset / idx / capacity / ring bookkeeping as host integers, exactly as
// Libraries/MLXLMCommon/KVCache.swift keeps them), device page storage, and the
// extern "C" surface declared in include/kvhip.h.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "kvhip_internal.hpp"

using namespace kvhip;

namespace {

thread_local std::string g_err;
thread_local bool g_has_err = false;
// per calling thread, like the error state: caches driven from different threads do not share them
thread_local int g_policy = 0;
thread_local int g_last_kernel = -1;
bool g_inited = false;

// code widths of MLX's affine quantization
bool affine_bits_ok(int bits) { return bits == 2 || bits == 3 || bits == 4 || bits == 5 || bits == 6 || bits == 8; }

kvhip_status fail(kvhip_status code, const std::string &msg) {
    g_err = msg;
    g_has_err = true;
    return code;
}

#define KV_HIP(expr)                                                                         \
    do {                                                                                     \
        hipError_t e_ = (expr);                                                              \
        if (e_ != hipSuccess)                                                                \
            return fail(KVHIP_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_));   \
    } while (0)
// the same, running `cleanup` before the early return
#define KV_HIP_OR(expr, cleanup)                                                             \
    do {                                                                                     \
        hipError_t e_ = (expr);                                                              \
        if (e_ != hipSuccess) {                                                              \
            cleanup;                                                                         \
            return fail(KVHIP_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_));   \
        }                                                                                    \
    } while (0)
#define KV_TRY(expr)                         \
    do {                                     \
        kvhip_status s_ = (expr);            \
        if (s_ != KVHIP_OK) return s_;       \
    } while (0)

int elem_size(int dtype) { return dtype == KVHIP_F32 ? 4 : 2; }

// Fixed scratch of kvhip_cache_attend_static: the span partials of the attention kernels when the
// caller cannot allocate.  One copy per device, resident until the process ends.  In host code
// the array's name is only a handle for hipGetSymbolAddress; every use of its memory goes through
// the per-device address looked up in kvhip_init.
constexpr size_t SCRATCH_BYTES = (size_t)KVHIP_STATIC_SCRATCH_BYTES;
constexpr int MAX_DEVICES = 64;
float *g_scratch_ptr[MAX_DEVICES] = {};

}  // namespace

static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

// One device allocation backing a run of consecutive pages (all planes of those pages).
struct Slab {
    void *base = nullptr;
    int64_t first_page = 0, pages = 0;
    size_t bytes = 0;  // size of the allocation (at least what the pages need: it may come from the pool)
};

struct kvhip_cache {
    int kind = 0;
    // constructor arguments
    int step = 256;
    int64_t max_size = 0;
    int64_t keep = 0;
    int gs = 64, bits = 8;
    std::string origin = "modelNative";
    // reference bookkeeping
    int64_t offset = 0;
    int64_t idx = 0;
    bool has_buffers = false;  // the reference's `keys != nil`
    int64_t ref_len = 0;       // row extent of the reference's buffers
    int64_t presented = 0;     // key extent the last update returned
    // geometry, fixed by the first update / import / reserve
    bool has_geom = false;
    int B = 0, Hkv = 0;
    Store st;                  // st.pt = the page table in device memory
    // Head sizes of the caller's arrays.  The pages hold st.Dk / st.Dv, which are larger when the tuned kernels are
    // not built for the caller's sizes: rows are then stored zero-padded (zero key columns add nothing to a score,
    // zero value columns give output columns nobody reads), arrays are widened on the way in and narrowed on the
    // way out, and everything between works on the stored sizes.
    int Dk_user = 0, Dv_user = 0;
    void *pad_buf[4] = {nullptr, nullptr, nullptr, nullptr};  // widened keys, values, queries; outputs before narrowing
    size_t pad_bytes[4] = {0, 0, 0, 0};
    std::vector<Slab> slabs;   // the allocations behind the pages, in page order
    int64_t cap_pages = 0;     // pages allocated (= page-table entries in use)
    int64_t pt_cap = 0;        // entries the device page table has room for
    // rotating only: reference row -> physical slot, and slot occupancy
    std::vector<int32_t> rows;
    std::vector<uint8_t> used;
    int64_t cursor = 0;
    // rotating only: an open staged round (RotatingStagedKVCache.swift:12-132).  Staged rows
    // sit in spare slots of the same page store; the ring's own rows are untouched until commit.
    bool staging = false;
    std::vector<int32_t> staged;      // slots of the staged rows, in write order
    std::vector<int32_t> stage_view;  // slots of the presentation: trailing window ++ staged
    int64_t presented_live = 0;       // `presented` of the live ring when the round opened
    void *stage_tmp_k = nullptr, *stage_tmp_v = nullptr;  // dense copy of the rows a commit keeps
    size_t stage_tmp_rows = 0;
    const RopeDev *rope = nullptr;  // set for the duration of one update_rope call
    // scratch for attention
    float *ws = nullptr;
    size_t ws_bytes = 0;
    // buffers replaced by larger ones while work that reads them may still be in flight: kept
    // until the cache is freed (hipFree would wait for the whole device)
    std::vector<std::pair<void *, size_t>> parked;
    // the stream the cache's device work was last enqueued on: freeing the cache releases its
    // memory behind that work instead of waiting for it
    mutable hipStream_t last_stream = nullptr;
    mutable bool used_stream = false;

    int64_t cap_slots() const { return cap_pages * PAGE; }
    bool padded() const { return has_geom && (Dk_user != st.Dk || Dv_user != st.Dv); }
};

namespace {

// ---- page storage: slabs of pages behind a page table ------------------------------------------
// Device buffers that work in flight may still read (page tables and page slabs that were
// replaced, the memory of a freed cache) cannot be freed on the spot: hipFree waits for the whole
// device.  They are retired behind an event recorded on the stream of their last reader.  Once
// that event has completed (hipEventQuery: no waiting) a buffer moves to a free list, from which
// later allocations of a similar size are served instead of hipMalloc, so a loop that creates,
// grows and frees caches without ever calling a blocking entry point neither waits nor keeps
// growing the device's memory.  Buffers the free list holds beyond its limits, and everything on
// it when a blocking call runs (kvhip_sync, kvhip_cache_reserve, a hipMalloc that failed), are
// released with hipFree there.  Only the stream a cache was last used on is tracked: a caller who
// reads one cache on several streams orders them before kvhip_cache_free.
struct Buf {
    void *p = nullptr;
    size_t bytes = 0;  // 0: size not recorded, never reused
    int dev = 0;
};
struct Retired {
    hipEvent_t done;
    hipStream_t stream;  // where `done` was recorded: work enqueued there later runs after the buffers' last reader
    std::vector<Buf> bufs;
};
std::mutex g_retired_mu;
std::vector<Retired> g_retired;
std::vector<Buf> g_free;                          // finished with, kept for reuse
constexpr size_t POOL_MAX_BUFS = 64;              // what the free list may hold after a blocking call
constexpr size_t POOL_MAX_BYTES = (size_t)4 << 30;

int current_device() {
    int d = 0;
    if (hipGetDevice(&d) != hipSuccess) (void)hipGetLastError();
    return d;
}

void retire(std::vector<std::pair<void *, size_t>> &&ptrs, hipStream_t stream) {
    if (ptrs.empty()) return;
    Retired r;
    r.stream = stream;
    const int dev = current_device();
    for (auto &q : ptrs) r.bufs.push_back(Buf{q.first, q.second, dev});
    if (hipEventCreateWithFlags(&r.done, hipEventDisableTiming) != hipSuccess || hipEventRecord(r.done, stream) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipDeviceSynchronize();
        for (const Buf &b : r.bufs) (void)hipFree(b.p);
        return;
    }
    std::lock_guard<std::mutex> lock(g_retired_mu);
    g_retired.push_back(std::move(r));
}

// Moves retired buffers whose readers have finished to the free list.  Never waits.  (lock held)
void harvest_locked() {
    for (size_t i = 0; i < g_retired.size();) {
        if (hipEventQuery(g_retired[i].done) != hipSuccess) {
            (void)hipGetLastError();
            ++i;
            continue;
        }
        for (const Buf &b : g_retired[i].bufs) g_free.push_back(b);
        (void)hipEventDestroy(g_retired[i].done);
        g_retired[i] = std::move(g_retired.back());
        g_retired.pop_back();
    }
}

// hipMalloc, or a finished buffer of at least `bytes` and at most 1.5 times that from the free list.
// `got` receives the size of what was handed out.  Only enqueue-free work: usable on the hot path.
// `same_stream`: the buffer will only be touched by work enqueued on that stream from now on, so a buffer retired
// behind earlier work of the same stream may be handed out before that work has finished (stream order keeps the
// new user behind the old reader): scratch that every call takes and gives back is then one buffer per stream
// however far the host runs ahead.
hipError_t pool_alloc(void **out, size_t bytes, size_t *got, const hipStream_t *same_stream = nullptr) {
    {
        std::lock_guard<std::mutex> lock(g_retired_mu);
        harvest_locked();
        const int dev = current_device();
        if (same_stream) {
            for (size_t i = 0; i < g_retired.size(); ++i) {
                Retired &r = g_retired[i];
                if (r.stream != *same_stream) continue;
                for (size_t j = 0; j < r.bufs.size(); ++j) {
                    const Buf &b = r.bufs[j];
                    if (b.dev != dev || b.bytes < bytes || b.bytes > bytes + bytes / 2) continue;
                    *out = b.p;
                    *got = b.bytes;
                    r.bufs[j] = r.bufs.back();
                    r.bufs.pop_back();
                    if (r.bufs.empty()) {
                        (void)hipEventDestroy(r.done);
                        g_retired[i] = std::move(g_retired.back());
                        g_retired.pop_back();
                    }
                    return hipSuccess;
                }
            }
        }
        int best = -1;
        for (size_t i = 0; i < g_free.size(); ++i) {
            const Buf &b = g_free[i];
            if (b.dev != dev || b.bytes < bytes || b.bytes > bytes + bytes / 2) continue;
            if (best < 0 || b.bytes < g_free[best].bytes) best = (int)i;
        }
        if (best >= 0) {
            *out = g_free[best].p;
            *got = g_free[best].bytes;
            g_free[best] = g_free.back();
            g_free.pop_back();
            return hipSuccess;
        }
    }
    *got = bytes;
    return hipMalloc(out, bytes);
}

// Releases what the free list holds beyond its limits (`all`: everything).  Blocks (hipFree does): never on
// the hot path.
void reap_retired(bool all = false) {
    std::vector<Buf> drop;
    {
        std::lock_guard<std::mutex> lock(g_retired_mu);
        harvest_locked();
        size_t total = 0;
        std::vector<Buf> keep;
        // the most recently finished buffers are the likeliest to be asked for again
        for (size_t i = g_free.size(); i-- > 0;) {
            const Buf &b = g_free[i];
            if (!all && b.bytes > 0 && keep.size() < POOL_MAX_BUFS && total + b.bytes <= POOL_MAX_BYTES) {
                keep.push_back(b);
                total += b.bytes;
            } else {
                drop.push_back(b);
            }
        }
        g_free.swap(keep);
    }
    for (const Buf &b : drop) (void)hipFree(b.p);
}

// The same when `stream` has nothing in flight (then hipFree has little to wait for).
void reap_if_idle(hipStream_t stream) {
    if (hipStreamQuery(stream) == hipSuccess) reap_retired();
    else (void)hipGetLastError();
}

size_t align256(size_t n) { return (n + 255) / 256 * 256; }

// Gives up the cache's pages and page table: freed at once when nothing in flight can read them
// (`drained`), otherwise retired behind the work enqueued on `stream` so far.
void drop_pages(kvhip_cache *c, hipStream_t stream, bool drained) {
    std::vector<std::pair<void *, size_t>> ptrs;
    for (const Slab &sl : c->slabs) ptrs.push_back({sl.base, sl.bytes});
    if (c->st.pt) ptrs.push_back({const_cast<PageEntry *>(c->st.pt), (size_t)0});
    c->slabs.clear();
    c->st.pt = nullptr;
    c->cap_pages = 0;
    c->pt_cap = 0;
    if (drained) {
        for (auto &q : ptrs) (void)hipFree(q.first);
    } else {
        retire(std::move(ptrs), stream);
    }
}

// The head sizes a cache stores for the caller's (Dk, Dv).  The tuned attention kernels are built for 16-bit caches
// with one head size of 64, 96, 128 or 256 (80 too when not quantized) and for keys of 192 with values of 128; any
// other pair up to 256 is stored zero-padded to the next of 64 / 96 / 128 / 256 that holds both (and that the
// group size divides).  float32 caches and head sizes above 256 are stored as they are (plain kernel).
void stored_head_sizes(int kind, int gs, int dtype, int Dk, int Dv, int &Pk, int &Pv) {
    Pk = Dk;
    Pv = Dv;
    if (dtype != KVHIP_F16 && dtype != KVHIP_BF16) return;
    if (Dk == 192 && Dv == 128) return;
    const bool q = kind == KVHIP_KIND_QUANTIZED;
    if (Dk == Dv && (Dk == 64 || Dk == 96 || Dk == 128 || Dk == 256 || (!q && Dk == 80))) return;
    const int m = std::max(Dk, Dv);
    for (int p : {64, 96, 128, 256})
        if (p >= m && (!q || (gs > 0 && p % gs == 0))) {
            Pk = Pv = p;
            return;
        }
}

// Dk / Dv: the head sizes of the caller's arrays
kvhip_status set_geometry(kvhip_cache *c, int B, int Hkv, int Dk, int Dv, int dtype) {
    if (B <= 0 || Hkv <= 0 || Dk <= 0 || Dv <= 0) return fail(KVHIP_ERR_INVALID_ARG, "non-positive shape");
    if (dtype != KVHIP_F16 && dtype != KVHIP_BF16 && dtype != KVHIP_F32)
        return fail(KVHIP_ERR_INVALID_ARG, "cache dtype must be float16, bfloat16 or float32");
    if ((int64_t)B * Hkv > 65535) return fail(KVHIP_ERR_UNSUPPORTED, "B * Hkv above 65535");
    if (c->has_geom) {
        const Store &s = c->st;
        if (s.BH != B * Hkv || c->B != B || c->Dk_user != Dk || c->Dv_user != Dv || s.dtype != dtype)
            return fail(KVHIP_ERR_INVALID_ARG, "shape or dtype differs from what this cache already holds");
        return KVHIP_OK;
    }
    if (c->kind == KVHIP_KIND_QUANTIZED && c->gs > 0 && (Dk % c->gs || Dv % c->gs))
        return fail(KVHIP_ERR_INVALID_ARG, "head dim not divisible by the group size");
    Store &s = c->st;
    s = Store();
    c->B = B;
    c->Hkv = Hkv;
    c->Dk_user = Dk;
    c->Dv_user = Dv;
    stored_head_sizes(c->kind, c->gs, dtype, Dk, Dv, Dk, Dv);  // from here on: the stored sizes
    s.BH = B * Hkv;
    s.Dk = Dk;
    s.Dv = Dv;
    s.dtype = dtype;
    s.es = elem_size(dtype);
    if (c->kind == KVHIP_KIND_QUANTIZED) {
        if (!affine_bits_ok(c->bits))
            return fail(KVHIP_ERR_UNSUPPORTED, "affine KV quantization is implemented for 2, 3, 4, 5, 6 and 8 bits");
        if (Dk % c->gs || Dv % c->gs) return fail(KVHIP_ERR_INVALID_ARG, "head dim not divisible by the group size");
        s.bits = c->bits;
        s.gs = c->gs;
        s.k_row = (uint32_t)(Dk * c->bits / 8);
        s.k_cell = s.k_row * PAGE;
        s.v_cell = (uint32_t)(Dv * c->bits / 8) * PAGE;
        s.ksb_row = (uint32_t)(Dk / c->gs * 2 * s.es);
        s.vsb_row = (uint32_t)(Dv / c->gs * 2 * s.es);
        s.ksb_cell = s.ksb_row * PAGE;
        s.vsb_cell = s.vsb_row * PAGE;
    } else {
        // K rows are laid out in whole 16-byte chunks (the interleaved tile of kvhip_internal.hpp)
        s.k_row = (uint32_t)((Dk * s.es + 15) / 16 * 16);
        s.k_cell = s.k_row * PAGE;
        s.v_cell = (uint32_t)(Dv * s.es) * PAGE;
    }
    c->has_geom = true;
    return KVHIP_OK;
}

// Make room for `slots` physical slots.  Pages are appended: one new allocation backs the new
// pages, their entries are added to the page table by a small kernel on `stream`, and nothing
// that was written moves or is copied.  hipMalloc does not wait for work in flight, so the call
// only enqueues (the reference re-concatenates every buffer instead, KVCache.swift:419-435,
// :704-728, :981-989).  When the page table itself is full, a larger one is allocated and the old
// entries are copied into it on the stream (32 bytes per page); the old table is retired.
kvhip_status ensure_slots(kvhip_cache *c, int64_t slots, hipStream_t stream, bool exact = false) {
    const int64_t need = (slots + PAGE - 1) / PAGE;
    if (need <= c->cap_pages) return KVHIP_OK;
    int64_t pages = need;
    if (!exact && c->cap_pages > 0) pages = std::max(need, c->cap_pages + (c->cap_pages + 1) / 2);
    if (pages > ((int64_t)1 << 22)) return fail(KVHIP_ERR_UNSUPPORTED, "cache longer than 2^30 rows");
    const Store &st = c->st;
    const size_t BH = st.BH;
    if (pages > c->pt_cap) {
        int64_t cap = std::max<int64_t>(c->pt_cap * 2, 64);
        while (cap < pages) cap *= 2;
        void *npt = nullptr;
        KV_HIP(hipMalloc(&npt, (size_t)cap * sizeof(PageEntry)));  // (a few KB: not worth the pool)
        if (c->cap_pages > 0)
            KV_HIP_OR(launch_copy_bytes(npt, st.pt, (size_t)c->cap_pages * sizeof(PageEntry), stream), (void)hipFree(npt));
        if (st.pt) retire({{const_cast<PageEntry *>(st.pt), (size_t)0}}, stream);
        c->st.pt = static_cast<PageEntry *>(npt);
        c->pt_cap = cap;
    }
    // one allocation for the new pages: [K cells | K pairs | V cells | V pairs], each part page-major
    const int64_t add = pages - c->cap_pages;
    const size_t stride[4] = {BH * st.k_cell, BH * st.v_cell, BH * st.ksb_cell, BH * st.vsb_cell};
    const size_t part[4] = {align256(stride[0] * add), align256(stride[1] * add), align256(stride[2] * add), align256(stride[3] * add)};
    const size_t bytes = part[0] + part[1] + part[2] + part[3];
    void *base = nullptr;
    size_t got = bytes;
    hipError_t e = pool_alloc(&base, bytes, &got);
    if (e != hipSuccess) {  // memory of freed caches may still be waiting for its release: wait for it and retry
        (void)hipGetLastError();
        (void)hipDeviceSynchronize();
        reap_retired(true);
        got = bytes;
        e = hipMalloc(&base, bytes);
    }
    if (e != hipSuccess)
        return fail(KVHIP_ERR_HIP, std::string("hipMalloc of ") + std::to_string(bytes) + " bytes of cache pages failed: " + hipGetErrorString(e));
    // packed V words are merged read-modify-write: new pages start from zero
    KV_HIP_OR(launch_fill_zero(base, bytes, stream), (void)hipFree(base));
    PageEntry first;
    char *p = static_cast<char *>(base);
    first.k = p;
    first.v = p + part[0];
    first.ksb = st.ksb_cell ? p + part[0] + part[1] : nullptr;
    first.vsb = st.vsb_cell ? p + part[0] + part[1] + part[2] : nullptr;
    KV_HIP_OR(launch_set_pages(const_cast<PageEntry *>(st.pt), (int)c->cap_pages, (int)add, first, stride, stream), (void)hipFree(base));
    Slab sl;
    sl.base = base;
    sl.first_page = c->cap_pages;
    sl.pages = add;
    sl.bytes = got;
    c->slabs.push_back(sl);
    c->cap_pages = pages;
    if (c->kind == KVHIP_KIND_ROTATING) c->used.resize((size_t)c->cap_slots(), 0);
    return KVHIP_OK;
}

// Scratch of the attention kernels.  A larger one replaces it without waiting for the device:
// the old buffer stays allocated until the cache is freed.
kvhip_status ensure_ws(kvhip_cache *c, size_t bytes, hipStream_t) {
    if (bytes <= c->ws_bytes) return KVHIP_OK;
    const size_t want = std::max(bytes + bytes / 4, 2 * c->ws_bytes);
    void *p = nullptr;
    size_t got = want;
    KV_HIP(pool_alloc(&p, want, &got));
    if (c->ws) c->parked.push_back({c->ws, c->ws_bytes});
    c->ws = static_cast<float *>(p);
    c->ws_bytes = got;
    return KVHIP_OK;
}

// A cache that stores padded rows: the caller's dense array `src` (rows of `user_d` elements) widened into the
// cache's buffer number `which` (rows of `stored_d` elements, the added columns zero); `*out` is what the kernels read.
kvhip_status ensure_pad_buf(kvhip_cache *c, int which, size_t need) {
    if (need <= c->pad_bytes[which]) return KVHIP_OK;
    void *p = nullptr;
    size_t got = need;
    KV_HIP(pool_alloc(&p, std::max(need + need / 4, 2 * c->pad_bytes[which]), &got));
    if (c->pad_buf[which]) c->parked.push_back({c->pad_buf[which], c->pad_bytes[which]});  // (work in flight may read it)
    c->pad_buf[which] = p;
    c->pad_bytes[which] = got;
    return KVHIP_OK;
}

kvhip_status widen_rows(kvhip_cache *c, int which, const void *src, size_t rows, int user_d, int stored_d,
                        hipStream_t s, const void **out) {
    *out = src;
    if (user_d == stored_d) return KVHIP_OK;
    KV_TRY(ensure_pad_buf(c, which, rows * (size_t)stored_d * c->st.es));
    KV_HIP(launch_repitch_rows(c->pad_buf[which], (size_t)stored_d * c->st.es, src, (size_t)user_d * c->st.es, rows, s));
    *out = c->pad_buf[which];
    return KVHIP_OK;
}

// ---- run tables ------------------------------------------------------------
struct RunList {
    std::vector<int32_t> row0, phys0, len;
    size_t size() const { return row0.size(); }
};

RunList runs_of(const int32_t *slots, int64_t n) {
    RunList r;
    for (int64_t i = 0; i < n;) {
        int64_t j = i + 1;
        while (j < n && slots[j] == slots[j - 1] + 1) ++j;
        r.row0.push_back((int32_t)i);
        r.phys0.push_back(slots[i]);
        r.len.push_back((int32_t)(j - i));
        i = j;
    }
    return r;
}

Runs pack_runs(const RunList &rl, size_t first, size_t count) {
    Runs r;
    r.n = (int32_t)count;
    for (size_t i = 0; i < (size_t)MAXRUNS; ++i) {
        const bool live = i < count;
        r.row0[i] = live ? rl.row0[first + i] : 0;
        r.phys0[i] = live ? rl.phys0[first + i] : 0;
        r.len[i] = live ? rl.len[first + i] : 0;
    }
    return r;
}

Runs identity_runs(int64_t n) {
    RunList rl;
    if (n > 0) {
        rl.row0.push_back(0);
        rl.phys0.push_back(0);
        rl.len.push_back((int32_t)n);
    }
    return pack_runs(rl, 0, rl.size());
}

// Dense export of the rows named by `slots` (any order) into [BH, n, D] arrays.
// dense arrays of the stored head sizes
kvhip_status export_slots_stored(const kvhip_cache *c, const int32_t *slots, int64_t n, void *dk, void *dv,
                                 hipStream_t stream) {
    const RunList rl = runs_of(slots, n);
    for (size_t first = 0; first < rl.size(); first += MAXRUNS) {
        const size_t cnt = std::min((size_t)MAXRUNS, rl.size() - first);
        const Runs r = pack_runs(rl, first, cnt);
        const int begin = rl.row0[first];
        const int end = rl.row0[first + cnt - 1] + rl.len[first + cnt - 1];
        KV_HIP(launch_export_fp(c->st, r, begin, end - begin, 0, (int)n, dk, dv, stream));
    }
    return KVHIP_OK;
}

// dense arrays of the caller's head sizes (a cache that stores padded rows exports into a buffer of the stored
// width first and narrows that; the buffer is handed back behind the stream's work)
kvhip_status export_slots(const kvhip_cache *c, const int32_t *slots, int64_t n, void *dk, void *dv,
                          hipStream_t stream) {
    if (!c->padded() || n <= 0) return export_slots_stored(c, slots, n, dk, dv, stream);
    const Store &st = c->st;
    const size_t rows = (size_t)st.BH * (size_t)n;
    void *tk = nullptr, *tv = nullptr;
    size_t gk = 0, gv = 0;
    if (dk) KV_HIP(pool_alloc(&tk, rows * st.Dk * st.es, &gk));
    if (dv) {
        const hipError_t e = pool_alloc(&tv, rows * st.Dv * st.es, &gv);
        if (e != hipSuccess) {
            if (tk) (void)hipFree(tk);
            KV_HIP(e);
        }
    }
    kvhip_status r = export_slots_stored(c, slots, n, tk, tv, stream);
    if (r == KVHIP_OK && tk && launch_repitch_rows(dk, (size_t)c->Dk_user * st.es, tk, (size_t)st.Dk * st.es, rows, stream) != hipSuccess)
        r = fail(KVHIP_ERR_HIP, "narrowing the exported keys failed");
    if (r == KVHIP_OK && tv && launch_repitch_rows(dv, (size_t)c->Dv_user * st.es, tv, (size_t)st.Dv * st.es, rows, stream) != hipSuccess)
        r = fail(KVHIP_ERR_HIP, "narrowing the exported values failed");
    std::vector<std::pair<void *, size_t>> tmp;
    if (tk) tmp.push_back({tk, gk});
    if (tv) tmp.push_back({tv, gv});
    retire(std::move(tmp), stream);
    return r;
}

// ---- rotating: physical slot management ---------------------------------------
kvhip_status ring_alloc(kvhip_cache *c, int64_t n, std::vector<int32_t> &out, hipStream_t stream) {
    int64_t live = 0;
    for (uint8_t u : c->used) live += u;
    if (live + n > c->cap_slots()) KV_TRY(ensure_slots(c, live + n, stream));
    const int64_t C = c->cap_slots();
    int64_t p = c->cursor % C;
    for (int64_t got = 0, scanned = 0; got < n; ++scanned) {
        if (scanned > 2 * C) return fail(KVHIP_ERR_INTERNAL, "ring slot allocation found no free slot");
        if (!c->used[(size_t)p]) {
            c->used[(size_t)p] = 1;
            out.push_back((int32_t)p);
            ++got;
        }
        p = (p + 1) % C;
    }
    c->cursor = p;
    return KVHIP_OK;
}

void ring_release(kvhip_cache *c, const std::vector<int32_t> &rows, size_t lo, size_t hi) {
    for (size_t i = lo; i < hi && i < rows.size(); ++i) c->used[(size_t)rows[i]] = 0;
}

// `trim(trimSize:_:)` (KVCache.swift:576-590) on the row map
void ring_front_trim(kvhip_cache *c, int64_t trim) {
    if (trim <= 0) return;
    const size_t keep = (size_t)std::min<int64_t>(c->keep, (int64_t)c->rows.size());
    const size_t cut_hi = std::min(c->rows.size(), keep + (size_t)trim);
    ring_release(c, c->rows, keep, cut_hi);
    c->rows.erase(c->rows.begin() + keep, c->rows.begin() + cut_hi);
}

// `temporalOrder(_:)` (KVCache.swift:592-606) as a permutation of the row map
std::vector<int32_t> temporal_order(const kvhip_cache *c, std::vector<int32_t> *dropped = nullptr) {
    const std::vector<int32_t> &a = c->rows;
    const int64_t len = (int64_t)a.size();
    if (c->idx == len) return a;
    std::vector<int32_t> o;
    if (c->idx < c->offset) {
        const int64_t k = std::min<int64_t>(std::max<int64_t>(c->keep, 0), len);
        const int64_t i = std::min<int64_t>(std::max<int64_t>(c->idx, k), len);
        o.insert(o.end(), a.begin(), a.begin() + k);
        o.insert(o.end(), a.begin() + i, a.end());
        if (i > k) o.insert(o.end(), a.begin() + k, a.begin() + i);
        return o;
    }
    const int64_t i = std::min<int64_t>(std::max<int64_t>(c->idx, 0), len);
    o.assign(a.begin(), a.begin() + i);
    if (dropped) dropped->assign(a.begin() + i, a.end());
    return o;
}

// Write `n` new rows (src rows [src0, src0+n) of an [BH, L, D] pair) to the given slots.
kvhip_status write_rows(kvhip_cache *c, const void *keys, const void *values, int L, int src0,
                        const int32_t *slots, int64_t n, hipStream_t stream) {
    const RunList rl = runs_of(slots, n);
    for (size_t i = 0; i < rl.size(); ++i) {
        if (c->kind == KVHIP_KIND_QUANTIZED)
            KV_HIP(launch_append_quant(c->st, keys, values, L, src0 + rl.row0[i], rl.phys0[i], rl.len[i], stream, c->rope));
        else
            KV_HIP(launch_append_fp(c->st, keys, values, L, src0 + rl.row0[i], rl.phys0[i], rl.len[i], stream, c->rope));
    }
    return KVHIP_OK;
}

// Gather every live row (ring rows, then staged rows) into slot order in a fresh store, so
// that later launches see single runs.
kvhip_status compact_store(kvhip_cache *c, hipStream_t stream) {
    std::vector<int32_t> all(c->rows);
    all.insert(all.end(), c->staged.begin(), c->staged.end());
    const RunList rl = runs_of(all.data(), (int64_t)all.size());
    kvhip_cache tmp;
    tmp.kind = KVHIP_KIND_SIMPLE;  // plain page store: no slot occupancy to size
    tmp.has_geom = true;
    tmp.B = c->B;
    tmp.Hkv = c->Hkv;
    tmp.st = c->st;
    tmp.st.pt = nullptr;
    kvhip_status st = ensure_slots(&tmp, c->cap_slots(), stream, true);
    for (size_t first = 0; st == KVHIP_OK && first < rl.size(); first += MAXRUNS) {
        const size_t cnt = std::min((size_t)MAXRUNS, rl.size() - first);
        const hipError_t e = launch_compact_fp(c->st, pack_runs(rl, first, cnt), tmp.st, (int)all.size(), stream);
        if (e != hipSuccess) st = fail(KVHIP_ERR_HIP, std::string("ring gather failed: ") + hipGetErrorString(e));
    }
    if (st != KVHIP_OK) {
        drop_pages(&tmp, stream, false);
        return st;
    }
    // the old pages are retired behind the gather that reads them; the host does not wait
    drop_pages(c, stream, false);
    c->slabs.swap(tmp.slabs);
    c->st.pt = tmp.st.pt;
    c->cap_pages = tmp.cap_pages;
    c->pt_cap = tmp.pt_cap;
    std::fill(c->used.begin(), c->used.end(), 0);
    for (size_t i = 0; i < all.size(); ++i) c->used[i] = 1;
    for (size_t i = 0; i < c->rows.size(); ++i) c->rows[i] = (int32_t)i;
    for (size_t i = 0; i < c->staged.size(); ++i) c->staged[i] = (int32_t)(c->rows.size() + i);
    c->cursor = (int64_t)all.size();
    return KVHIP_OK;
}

// If the ring's rows are scattered over more runs than a kernel takes, compact.
// `steady`: a full ring taking single tokens.  Its rows keep their slots from now on, so the slots that the prompt
// chunks before it left unused inside the span of the rows -- every decode step would stream their tiles and drop
// them -- are squeezed out once (a gather into fresh pages, enqueued like the rest): at a 4096-row window behind
// 512-row chunks the decode kernel read 88 MB per step for 67 MB of rows.
kvhip_status ring_compact_if_needed(kvhip_cache *c, hipStream_t stream, bool steady = false) {
    const RunList rl = runs_of(c->rows.data(), (int64_t)c->rows.size());
    if (rl.size() > (size_t)MAXRUNS) return compact_store(c, stream);
    if (steady && c->staged.empty()) {
        int64_t span = 0;
        for (size_t i = 0; i < rl.size(); ++i) span = std::max<int64_t>(span, rl.phys0[i] + rl.len[i]);
        const int64_t unused = span - (int64_t)c->rows.size();
        if (unused >= TILE && unused * 8 >= span) return compact_store(c, stream);
    }
    return KVHIP_OK;
}

// ---- the three update paths ----------------------------------------------------
// `launch` false: everything but the append itself (pages, counters); the caller enqueues the
// write of rows [offset - L, offset) some other way.
kvhip_status update_simple(kvhip_cache *c, const void *k, const void *v, int L, hipStream_t stream, bool launch = true) {
    // KVCache.swift:404-447
    const int64_t prev = c->offset;
    int64_t ref_len = c->ref_len;
    if (!c->has_buffers || prev + L > c->ref_len) {
        const int64_t n_steps = (c->step + L - 1) / c->step;
        const int64_t grow = n_steps * c->step;
        ref_len = c->has_buffers ? ((prev % c->step) != 0 ? prev : c->ref_len) + grow : grow;
    }
    KV_TRY(ensure_slots(c, prev + L, stream));
    if (launch) {
        if (c->kind == KVHIP_KIND_QUANTIZED) KV_HIP(launch_append_quant(c->st, k, v, L, 0, (int)prev, L, stream, c->rope));
        else KV_HIP(launch_append_fp(c->st, k, v, L, 0, (int)prev, L, stream, c->rope));
    }
    // the host counters move only once the device work is enqueued
    c->ref_len = ref_len;
    c->has_buffers = true;
    c->offset = prev + L;
    c->presented = c->offset;
    return KVHIP_OK;
}

// deferred_slot (single-token steps only): the row is not written here; its physical slot is handed back and
// the caller sees to the write (the decode kernel takes it along).
kvhip_status update_rotating(kvhip_cache *c, const void *k, const void *v, int L, hipStream_t stream,
                             int32_t *deferred_slot = nullptr) {
    const int64_t M = c->max_size;
    if (L == 1) {
        // updateInPlace, KVCache.swift:684-740
        const int64_t prev = c->offset;
        if (!c->has_buffers || (prev >= c->ref_len && c->ref_len < M)) {
            const int64_t new_size = std::min<int64_t>(c->step, M - prev);
            if (new_size > 0) KV_TRY(ring_alloc(c, new_size, c->rows, stream));
            c->has_buffers = true;
            c->idx = prev;
        }
        const int64_t trim = (int64_t)c->rows.size() - M;
        if (trim > 0) {
            ring_front_trim(c, trim);
            c->idx = M;
        }
        if (c->idx == M) c->idx = c->keep;
        c->ref_len = (int64_t)c->rows.size();
        if (c->idx < 0 || c->idx >= c->ref_len)
            return fail(KVHIP_ERR_STATE, "RotatingKVCache write cursor lies outside its buffer");
        KV_TRY(ring_compact_if_needed(c, stream, c->ref_len == M && !c->staging));
        const int32_t slot = c->rows[(size_t)c->idx];
        if (deferred_slot) *deferred_slot = slot;
        else KV_HIP(launch_append_fp(c->st, k, v, 1, 0, slot, 1, stream, c->rope));
        c->offset += 1;
        c->idx += 1;
        c->presented = c->offset < M ? c->offset : c->ref_len;
        return KVHIP_OK;
    }
    // updateConcat, KVCache.swift:660-682
    if (!c->has_buffers) {
        KV_TRY(ring_alloc(c, L, c->rows, stream));
        c->has_buffers = true;
        KV_TRY(write_rows(c, k, v, L, 0, c->rows.data(), L, stream));
    } else {
        std::vector<int32_t> dropped;
        std::vector<int32_t> ordered = temporal_order(c, &dropped);
        for (int32_t s : dropped) c->used[(size_t)s] = 0;
        c->rows.swap(ordered);
        c->idx = (int64_t)c->rows.size();
        ring_front_trim(c, c->idx - M + 1);
        const size_t base = c->rows.size();
        KV_TRY(ring_alloc(c, L, c->rows, stream));
        KV_TRY(write_rows(c, k, v, L, 0, c->rows.data() + base, L, stream));
    }
    c->offset += L;
    c->ref_len = (int64_t)c->rows.size();
    c->idx = c->ref_len;
    c->presented = c->ref_len;
    return ring_compact_if_needed(c, stream);
}

// rows of the current presentation as (slot list or identity)
kvhip_status presented_runs(const kvhip_cache *c, Runs &runs, int &slots_span) {
    if (c->kind != KVHIP_KIND_ROTATING) {
        runs = identity_runs(c->presented);
        slots_span = (int)c->presented;
        return KVHIP_OK;
    }
    const bool staged_view = c->staging && !c->stage_view.empty();
    const std::vector<int32_t> &list = staged_view ? c->stage_view : c->rows;
    const RunList rl = runs_of(list.data(), std::min<int64_t>(c->presented, (int64_t)list.size()));
    if (rl.size() > (size_t)MAXRUNS) return fail(KVHIP_ERR_INTERNAL, "ring presentation not compacted");
    runs = pack_runs(rl, 0, rl.size());
    slots_span = 0;
    for (size_t i = 0; i < rl.size(); ++i) slots_span = std::max(slots_span, rl.phys0[i] + rl.len[i]);
    return KVHIP_OK;
}

// `logicalView(tail:)` (KVCache.swift:631-658) as a list of slots
std::vector<int32_t> logical_rows(const kvhip_cache *c, int64_t tail) {
    std::vector<int32_t> ordered = temporal_order(c);
    const int64_t available = (int64_t)ordered.size();
    const int64_t requested = std::min(std::max<int64_t>(tail, 0), available);
    const int64_t bound = std::max(requested, std::min<int64_t>(c->keep, available));
    const int64_t trim = available - bound;
    if (trim > 0) {
        const int64_t k = std::min<int64_t>(c->keep, available);
        ordered.erase(ordered.begin() + k, ordered.begin() + k + trim);
    }
    return ordered;
}

// `presentation(stagedKeys:stagedValues:)` (RotatingStagedKVCache.swift:78-91)
void stage_build_view(kvhip_cache *c) {
    c->stage_view.clear();
    const int64_t bound = std::min<int64_t>(c->offset, c->max_size - 1);
    if (bound > 0 && c->has_buffers) c->stage_view = logical_rows(c, bound);
    c->stage_view.insert(c->stage_view.end(), c->staged.begin(), c->staged.end());
}

// `RotatingStagedKVCache.update` (RotatingStagedKVCache.swift:41-47): the rows go to spare
// slots, the ring stays as it is, and the presentation is the trailing window plus
// everything staged so far -- read in place by the attention kernels, never concatenated.
kvhip_status stage_update(kvhip_cache *c, const void *k, const void *v, int L, hipStream_t stream) {
    const size_t base = c->staged.size();
    KV_TRY(ring_alloc(c, L, c->staged, stream));
    KV_TRY(write_rows(c, k, v, L, 0, c->staged.data() + base, L, stream));
    stage_build_view(c);
    if (runs_of(c->stage_view.data(), (int64_t)c->stage_view.size()).size() > (size_t)MAXRUNS) {
        KV_TRY(compact_store(c, stream));
        stage_build_view(c);
    }
    c->presented = (int64_t)c->stage_view.size();
    return KVHIP_OK;
}

int64_t state_rows(const kvhip_cache *c) {
    // KVCache.swift:449-460, :752-763, :1113-1130: sliced to offset when offset < extent
    if (!c->has_buffers) return 0;
    return c->offset < c->ref_len ? std::max<int64_t>(c->offset, 0) : c->ref_len;
}

hipStream_t S(void *s) { return reinterpret_cast<hipStream_t>(s); }
// the stream of a call that enqueues work reading or writing the cache's memory
hipStream_t S(const kvhip_cache *c, void *s) {
    c->last_stream = reinterpret_cast<hipStream_t>(s);
    c->used_stream = true;
    return c->last_stream;
}

kvhip_cache *new_cache_like(const kvhip_cache *c) {
    kvhip_cache *n = new kvhip_cache();
    n->kind = c->kind;
    n->step = c->step;
    n->max_size = c->max_size;
    n->keep = c->keep;
    n->gs = c->gs;
    n->bits = c->bits;
    return n;
}

}  // namespace

extern "C" {

const char *kvhip_version(void) { return "kvhip 0.1 (gfx950)"; }

const char *kvhip_last_error_message(void) { return g_has_err ? g_err.c_str() : nullptr; }

kvhip_status kvhip_init(int32_t device) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) return fail(KVHIP_ERR_NO_DEVICE, "no HIP device is visible");
    if (device < 0 || device >= n) return fail(KVHIP_ERR_INVALID_ARG, "device index out of range");
    KV_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    KV_HIP(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(KVHIP_ERR_NO_DEVICE, std::string("libkvhip is built for gfx950 only, found ") + prop.gcnArchName);
    if (device < MAX_DEVICES && !g_scratch_ptr[device]) {
        void *p = nullptr;
        KV_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));  // this device's copy of the array
        g_scratch_ptr[device] = static_cast<float *>(p);
    }
    g_inited = true;
    return KVHIP_OK;
}

kvhip_status kvhip_sync(void *stream) {
    KV_HIP(hipStreamSynchronize(S(stream)));
    reap_retired();
    return KVHIP_OK;
}

void kvhip_set_kernel_policy(int32_t policy) { g_policy = policy; }

int32_t kvhip_last_attend_kernel(void) { return g_last_kernel; }

void kvhip_profile_enable(int32_t every) { profile_enable(every); }

kvhip_status kvhip_profile_read(int32_t *out_launches, double *out_total_ms) {
    if (!out_launches || !out_total_ms) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    int n = 0;
    KV_HIP(profile_read(&n, out_total_ms));
    *out_launches = n;
    return KVHIP_OK;
}

kvhip_status kvhip_cache_create(const kvhip_config *cfg, kvhip_cache **out) {
    if (!cfg || !out) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (cfg->kind < 0 || cfg->kind > 2) return fail(KVHIP_ERR_INVALID_ARG, "unknown cache kind");
    kvhip_cache *c = new kvhip_cache();
    c->kind = cfg->kind;
    c->step = cfg->step > 0 ? cfg->step : 256;
    if (c->kind == KVHIP_KIND_ROTATING) {
        if (cfg->max_size <= 0) {
            delete c;
            return fail(KVHIP_ERR_INVALID_ARG, "RotatingKVCache requires a positive maxSize");
        }
        c->max_size = cfg->max_size;
        c->keep = std::max(0, cfg->keep);
    }
    if (c->kind == KVHIP_KIND_QUANTIZED) {
        c->step = 256;  // `private let step` fixed at 256, KVCache.swift:934
        c->gs = cfg->group_size > 0 ? cfg->group_size : 64;
        c->bits = cfg->bits > 0 ? cfg->bits : 8;
    }
    *out = c;
    return KVHIP_OK;
}

void kvhip_cache_free(kvhip_cache *c) {
    if (!c) return;
    // Work that reads the cache may still be in flight on the stream it was last used on.  Its
    // memory is handed to the retired list behind an event on that stream and released later,
    // so that dropping a cache (a conversion replacing it, the end of a round) does not make the
    // host wait for the device.
    std::vector<std::pair<void *, size_t>> ptrs;
    for (const Slab &sl : c->slabs) ptrs.push_back({sl.base, sl.bytes});
    if (c->st.pt) ptrs.push_back({const_cast<PageEntry *>(c->st.pt), (size_t)0});
    if (c->ws) ptrs.push_back({c->ws, c->ws_bytes});
    for (int i = 0; i < 4; ++i)
        if (c->pad_buf[i]) ptrs.push_back({c->pad_buf[i], c->pad_bytes[i]});
    if (c->stage_tmp_k) ptrs.push_back({c->stage_tmp_k, (size_t)0});
    if (c->stage_tmp_v) ptrs.push_back({c->stage_tmp_v, (size_t)0});
    for (auto &q : c->parked) ptrs.push_back(q);
    const hipStream_t stream = c->last_stream;
    const bool used = c->used_stream;
    delete c;
    if (ptrs.empty()) return;
    if (!used) {  // no device work ever touched it
        for (auto &q : ptrs) (void)hipFree(q.first);
        return;
    }
    retire(std::move(ptrs), stream);
    reap_if_idle(stream);
}

int64_t kvhip_cache_offset(const kvhip_cache *c) { return c ? c->offset : -1; }
int64_t kvhip_cache_idx(const kvhip_cache *c) { return c ? c->idx : -1; }
int64_t kvhip_cache_max_size(const kvhip_cache *c) { return (c && c->kind == KVHIP_KIND_ROTATING) ? c->max_size : -1; }
int32_t kvhip_cache_group_size(const kvhip_cache *c) { return c ? c->gs : -1; }
int32_t kvhip_cache_bits(const kvhip_cache *c) { return c ? c->bits : -1; }
int64_t kvhip_cache_capacity(const kvhip_cache *c) { return c ? c->ref_len : -1; }
int64_t kvhip_cache_presented_length(const kvhip_cache *c) { return c ? c->presented : -1; }
int64_t kvhip_cache_device_rows(const kvhip_cache *c) { return c ? c->cap_slots() : -1; }
int64_t kvhip_cache_slot_span(const kvhip_cache *c) {
    if (!c) return -1;
    if (c->kind != KVHIP_KIND_ROTATING) return c->presented;
    int64_t span = 0;
    for (int32_t slot : c->rows) span = std::max<int64_t>(span, (int64_t)slot + 1);
    return span;
}

int32_t kvhip_cache_is_trimmable(const kvhip_cache *c, int64_t after) {
    if (!c) return 0;
    if (c->kind == KVHIP_KIND_ROTATING) return c->offset + after < c->max_size;  // KVCache.swift:821-823
    return 1;
}

int64_t kvhip_cache_trim(kvhip_cache *c, int64_t n) {
    if (!c) return 0;
    const int64_t t = std::min(c->offset, n);  // KVCache.swift:474-478, :826-831, :1171-1175
    c->offset -= t;
    if (c->kind == KVHIP_KIND_ROTATING) c->idx -= t;
    return t;
}

kvhip_status kvhip_cache_set_offset(kvhip_cache *c, int64_t offset) {
    if (!c) return fail(KVHIP_ERR_INVALID_ARG, "null cache");
    c->offset = offset;
    return KVHIP_OK;
}

int32_t kvhip_resolved_group_size(int32_t requested, int32_t kd, int32_t vd) {
    // KVCache.swift:902-920
    requested = std::max(1, requested);
    int best = 0;
    for (int g : {32, 64, 128}) {
        if (kd % g || vd % g) continue;
        if (!best || std::abs(g - requested) < std::abs(best - requested)) best = g;
    }
    return best;
}

kvhip_status kvhip_cache_reserve(kvhip_cache *c, int32_t B, int32_t Hkv, int32_t Dk, int32_t Dv,
                                 int32_t dtype, int64_t tokens) {
    if (!c) return fail(KVHIP_ERR_INVALID_ARG, "null cache");
    if (c->kind == KVHIP_KIND_QUANTIZED && !c->has_buffers && c->offset == 0) {
        const int eff = kvhip_resolved_group_size(c->gs, Dk, Dv);
        if (!eff) return fail(KVHIP_ERR_STATE, "KV cache quantization requires head dimensions divisible by 32, 64 or 128");
        c->gs = eff;
    }
    KV_TRY(set_geometry(c, B, Hkv, Dk, Dv, dtype));
    reap_retired();
    KV_TRY(ensure_slots(c, tokens, nullptr, true));
    // the zero-fill of the new pages ran on the default stream: wait for it here, so that a
    // first update on any other (non-blocking) stream is ordered after it
    KV_HIP(hipStreamSynchronize(nullptr));
    return KVHIP_OK;
}

kvhip_status kvhip_cache_update(kvhip_cache *c, const void *keys, const void *values, int32_t B,
                                int32_t Hkv, int32_t L, int32_t Dk, int32_t Dv, int32_t dtype, void *stream) {
    if (!c || !keys || !values) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (L <= 0) return fail(KVHIP_ERR_INVALID_ARG, "update needs at least one new row");
    if (c->kind == KVHIP_KIND_QUANTIZED) {
        // KVCache.swift:1020-1037
        const int eff = kvhip_resolved_group_size(c->gs, Dk, Dv);
        if (!eff)
            return fail(KVHIP_ERR_STATE,
                        "KV cache quantization requires head dimensions divisible by one of the supported group sizes (32, 64, 128)");
        if (eff != c->gs && !c->has_buffers && c->offset == 0) {
            if (c->has_geom && c->cap_pages > 0) return fail(KVHIP_ERR_STATE, "group size changed after storage was reserved");
            c->gs = eff;
            c->has_geom = false;
        }
    }
    KV_TRY(set_geometry(c, B, Hkv, Dk, Dv, dtype));
    if (c->padded()) {  // rows of the stored head sizes, the added columns zero (a rotation reads its partners inside Dk)
        const size_t rows = (size_t)B * Hkv * L;
        KV_TRY(widen_rows(c, 0, keys, rows, Dk, c->st.Dk, S(c, stream), &keys));
        KV_TRY(widen_rows(c, 1, values, rows, Dv, c->st.Dv, S(c, stream), &values));
    }
    if (c->staging) return stage_update(c, keys, values, L, S(c, stream));
    if (c->kind == KVHIP_KIND_ROTATING) return update_rotating(c, keys, values, L, S(c, stream));
    return update_simple(c, keys, values, L, S(c, stream));
}

namespace {
// host description -> device description; `H` heads per batch row of the rotated array
kvhip_status rope_dev(const kvhip_rope *rope, int D, int H, int64_t pos0, const int32_t *batch_pos, RopeDev &r) {
    if (!rope) return fail(KVHIP_ERR_INVALID_ARG, "null rope description");
    if (rope->dims <= 0 || (rope->dims & 1) || rope->dims > D)
        return fail(KVHIP_ERR_INVALID_ARG, "rope dims must be even and at most the head dim");
    if (!rope->freqs && !(rope->base > 0.f)) return fail(KVHIP_ERR_INVALID_ARG, "rope base must be positive");
    r.dims = rope->dims;
    r.traditional = rope->traditional ? 1 : 0;
    r.scale = rope->scale;
    r.log_base_over_half = rope->freqs ? 0. : log((double)rope->base) / (double)(rope->dims / 2);
    r.freqs = rope->freqs;
    r.pos0 = (int32_t)pos0;
    r.batch_pos = batch_pos;
    r.H = H;
    return KVHIP_OK;
}
}  // namespace

kvhip_status kvhip_rope_apply(const kvhip_rope *rope, const void *x, void *out, int32_t B, int32_t H,
                              int32_t L, int32_t D, int32_t dtype, int64_t offset,
                              const int32_t *batch_offsets, void *stream) {
    if (!x || !out) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (B <= 0 || H <= 0 || L <= 0 || D <= 0 || D > 1024) return fail(KVHIP_ERR_INVALID_ARG, "shape out of range");
    if (dtype != KVHIP_F16 && dtype != KVHIP_BF16 && dtype != KVHIP_F32)
        return fail(KVHIP_ERR_INVALID_ARG, "rope needs a floating-point dtype");
    RopeDev r;
    KV_TRY(rope_dev(rope, D, H, offset, batch_offsets, r));
    KV_HIP(launch_rope_apply(r, x, out, B, H, L, D, dtype, S(stream)));
    return KVHIP_OK;
}

kvhip_status kvhip_cache_update_rope(kvhip_cache *c, const kvhip_rope *rope, const int32_t *batch_offsets,
                                     const void *keys, const void *values, int32_t B, int32_t Hkv, int32_t L,
                                     int32_t Dk, int32_t Dv, int32_t dtype, void *stream) {
    if (!c) return fail(KVHIP_ERR_INVALID_ARG, "null cache");
    RopeDev r;
    // `ropeOffset` is read before the write (Llama.swift:58-62); the staged wrapper's offset
    // counts its staged rows (RotatingStagedKVCache.swift:33-37)
    const int64_t pos0 = c->offset + (c->staging ? (int64_t)c->staged.size() : 0);
    KV_TRY(rope_dev(rope, Dk, Hkv, pos0, batch_offsets, r));
    c->rope = &r;
    const kvhip_status st = kvhip_cache_update(c, keys, values, B, Hkv, L, Dk, Dv, dtype, stream);
    c->rope = nullptr;
    return st;
}

kvhip_status kvhip_cache_fetch(const kvhip_cache *c, void *dk, void *dv, void *stream) {
    if (!c) return fail(KVHIP_ERR_INVALID_ARG, "null cache");
    if (c->kind == KVHIP_KIND_QUANTIZED)
        return fail(KVHIP_ERR_STATE, "`update` was called on `QuantizedKVCache`. Use `updateQuantized` instead.");
    if (c->staging && !c->stage_view.empty())
        return export_slots(c, c->stage_view.data(), (int64_t)c->stage_view.size(), dk, dv, S(c, stream));
    if (!c->has_buffers) return fail(KVHIP_ERR_STATE, "cache is empty");
    if (c->kind == KVHIP_KIND_ROTATING)
        return export_slots(c, c->rows.data(), c->presented, dk, dv, S(c, stream));
    std::vector<int32_t> ident((size_t)c->presented);
    for (size_t i = 0; i < ident.size(); ++i) ident[i] = (int32_t)i;
    return export_slots(c, ident.data(), c->presented, dk, dv, S(c, stream));
}

namespace {
// The cache's own workspace (grown with hipMalloc when a call needs more), or -- for callers that
// cannot allocate -- a fixed one the call must fit into.
kvhip_status bind_workspace(kvhip_cache *c, AttendArgs &a, size_t need, float *fixed, size_t fixed_bytes, hipStream_t s) {
    if (fixed) {
        if (need > fixed_bytes)
            return fail(KVHIP_ERR_UNSUPPORTED, "this call needs " + std::to_string(need) + " bytes of scratch, more than the " +
                                                   std::to_string(fixed_bytes) + " the allocation-free entry point holds");
        a.workspace = fixed;
        a.workspace_bytes = fixed_bytes;
        return KVHIP_OK;
    }
    KV_TRY(ensure_ws(c, need, s));
    a.workspace = c->ws;
    a.workspace_bytes = c->ws_bytes;
    return KVHIP_OK;
}

// A prompt chunk with many query rows per kv head over a quantized cache (attend_prefill_dequant_first): the cached
// rows are dequantized once into scratch pages of the cache dtype -- `MLX.dequantized`'s values, scale * code + bias
// in float32 rounded once -- and the chunk runs on the full-precision prefill tile, which needs no conversions in
// its loop.  The scratch (a page table, K pages, V pages) comes from the pool and goes back to it behind the call:
// calls on one stream share one buffer.  Returns KVHIP_ERR_HIP only for launch failures; when the scratch cannot be
// had, `*done` stays false and the caller runs the quantized tile.
// `valu`: head sizes above 256, which the tile is not built for -- the vector-ALU kernel runs over the scratch pages instead.
kvhip_status attend_dequant_first(kvhip_cache *c, const AttendArgs &a, hipStream_t s, bool *done, bool valu = false) {
    *done = false;
    Store t;
    t.BH = a.st.BH;
    t.Dk = a.st.Dk;
    t.Dv = a.st.Dv;
    t.dtype = a.st.dtype;
    t.es = a.st.es;
    t.k_row = (uint32_t)((t.Dk * t.es + 15) / 16 * 16);
    t.k_cell = t.k_row * PAGE;
    t.v_cell = (uint32_t)(t.Dv * t.es) * PAGE;
    const int64_t pages = ((int64_t)a.slots + PAGE - 1) / PAGE;
    const size_t BH = t.BH;
    const size_t ptb = align256((size_t)pages * sizeof(PageEntry)), kb = align256(BH * t.k_cell * pages), vb = align256(BH * t.v_cell * pages);
    void *base = nullptr;
    size_t got = 0;
    if (pool_alloc(&base, ptb + kb + vb, &got, &s) != hipSuccess) {
        (void)hipGetLastError();
        return KVHIP_OK;
    }
    std::vector<std::pair<void *, size_t>> give_back{{base, got}};
    PageEntry first;
    first.k = static_cast<char *>(base) + ptb;
    first.v = static_cast<char *>(base) + ptb + kb;
    const size_t stride[2] = {BH * t.k_cell, BH * t.v_cell};
    t.pt = static_cast<PageEntry *>(base);
    AttendArgs a2 = a;
    a2.st = t;
    kvhip_status st = KVHIP_OK;
    hipError_t e;
    if (t.es == 2) {
        e = launch_dequant_scratch(a.st, t, a.T, (int)pages, first, stride[0], stride[1], s);
    } else {  // float32 scales: the page table, then the element-wise pass over whole tiles (what lies past the
              // presented rows in the last tile is zeros or rows trimmed earlier: finite values the kernel weighs with 0)
        const size_t stride4[4] = {stride[0], stride[1], 0, 0};
        e = launch_set_pages(const_cast<PageEntry *>(t.pt), 0, (int)pages, first, stride4, s);
        const int rows_up = (int)std::min<int64_t>(pages * PAGE, ((int64_t)a.T + TILE - 1) / TILE * TILE);
        if (e == hipSuccess) e = launch_dequant_pages(a.st, t, rows_up, s);
    }
    if (e == hipSuccess) st = bind_workspace(c, a2, valu ? attend_valu_workspace(a2) : attend_prefill_workspace(a2), nullptr, 0, s);
    if (e == hipSuccess && st == KVHIP_OK) e = valu ? launch_attend_valu(a2, s) : launch_attend_prefill(a2, s);
    if (e == hipSuccess && st == KVHIP_OK && mask_may_leave_rows_without_keys(a2)) e = launch_rows_without_keys(a2, s);
    retire(std::move(give_back), s);
    if (e != hipSuccess) return fail(KVHIP_ERR_HIP, std::string("dequantize-first prefill: ") + hipGetErrorString(e));
    if (st != KVHIP_OK) return st;
    *done = true;
    return KVHIP_OK;
}

// new_k / new_v: the rows of a single-token step whose bookkeeping is done but whose write into physical
// slot `new_slot` is still owed; the decode kernel takes them along when it can, else they are
// appended by a launch of their own first.
kvhip_status attend_impl(kvhip_cache *c, const void *q, int32_t B, int32_t Hq, int32_t L, int32_t D, float scale,
                         const kvhip_mask *mask, void *out, void *stream, float *fixed, size_t fixed_bytes,
                         const void *new_k = nullptr, const void *new_v = nullptr, int32_t new_slot = -1) {
    if (!c || !q || !out) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    const bool staged_view = c->staging && !c->stage_view.empty();
    if (!c->has_geom || (!c->has_buffers && !staged_view) || c->presented <= 0)
        return fail(KVHIP_ERR_STATE, "attention over an empty cache");
    if (B != c->B || D != c->Dk_user) return fail(KVHIP_ERR_INVALID_ARG, "query shape does not match the cache");
    if (Hq <= 0 || Hq % c->Hkv) return fail(KVHIP_ERR_INVALID_ARG, "query heads must be a multiple of KV heads");
    if (L <= 0 || L > 65535) return fail(KVHIP_ERR_INVALID_ARG, "query length out of range");
    // A cache that stores padded rows: the queries are widened with zero columns and the kernels write output rows of
    // the stored width, which are narrowed at the end.  The allocation-free entry takes both buffers from the front of
    // its scratch.
    void *user_out = nullptr;
    const size_t q_rows = (size_t)B * Hq * L;
    if (c->padded()) {
        const size_t es = c->st.es;
        if (fixed) {
            const size_t qb = align256(q_rows * c->st.Dk * es), ob = align256(q_rows * c->st.Dv * es);
            if (qb + ob > fixed_bytes / 2)
                return fail(KVHIP_ERR_UNSUPPORTED, "the padded queries and outputs of this call do not fit the allocation-free entry point's scratch");
            char *base = reinterpret_cast<char *>(fixed);
            KV_HIP(launch_repitch_rows(base, (size_t)c->st.Dk * es, q, (size_t)D * es, q_rows, S(c, stream)));
            q = base;
            user_out = out;
            out = base + qb;
            fixed = reinterpret_cast<float *>(base + qb + ob);
            fixed_bytes -= qb + ob;
        } else {
            KV_TRY(widen_rows(c, 2, q, q_rows, D, c->st.Dk, S(c, stream), &q));
            KV_TRY(ensure_pad_buf(c, 3, q_rows * c->st.Dv * es));
            user_out = out;
            out = c->pad_buf[3];
        }
    }
    AttendArgs a;
    a.st = c->st;
    KV_TRY(presented_runs(c, a.runs, a.slots));
    a.q = q;
    a.out = out;
    a.B = B;
    a.Hq = Hq;
    a.Hkv = c->Hkv;
    a.L = L;
    a.T = (int)c->presented;
    a.scale = scale;
    if (mask) {
        MaskDev &m = a.mask;
        m.mode = mask->mode;
        if (m.mode < 0 || m.mode > 3) return fail(KVHIP_ERR_INVALID_ARG, "unknown mask mode");
        if (m.mode == KVHIP_MASK_ARRAY) {
            if (!mask->data) return fail(KVHIP_ERR_INVALID_ARG, "array mask without data");
            if (mask->key_len != a.T)
                return fail(KVHIP_ERR_INVALID_ARG, "array mask key extent differs from the presented length");
            if (mask->dtype != KVHIP_BOOL && mask->dtype != KVHIP_F16 && mask->dtype != KVHIP_BF16 && mask->dtype != KVHIP_F32)
                return fail(KVHIP_ERR_INVALID_ARG, "array mask dtype must be bool or a float type");
            m.dtype = mask->dtype;
            m.data = mask->data;
            m.sb = mask->stride_b;
            m.sh = mask->stride_h;
            m.sl = mask->stride_l;
        } else if (m.mode == KVHIP_MASK_WINDOW) {
            m.offset = mask->offset;
            m.window = mask->window;
            m.lengths = mask->lengths;
            m.left_pad = mask->left_pad;
        }
    }
    hipStream_t s = S(c, stream);
    a.workspace_cap = fixed ? fixed_bytes : 0;
    if (new_k) {
        if (g_policy != 1 && attend_decode_fuses_append(a)) {
            a.new_k = new_k;
            a.new_v = new_v;
            a.new_slot = new_slot;
        } else if (c->st.bits != 0) {
            KV_HIP(launch_append_quant(c->st, new_k, new_v, 1, 0, new_slot, 1, s, nullptr));
        } else {
            KV_HIP(launch_append_fp(c->st, new_k, new_v, 1, 0, new_slot, 1, s, nullptr));
        }
    }
    if (g_policy != 1 && attend_decode_supported(a)) {
        KV_TRY(bind_workspace(c, a, attend_decode_workspace(a), fixed, fixed_bytes, s));
        KV_HIP(launch_attend_decode(a, s));
        g_last_kernel = a.st.bits ? 1 : 2;
    } else if (g_policy != 1 && attend_prefill_supported(a)) {
        bool done = false;
        if (!fixed && g_policy != 2 && attend_prefill_dequant_first(a, g_policy == 3)) KV_TRY(attend_dequant_first(c, a, s, &done));
        if (!done) {
            KV_TRY(bind_workspace(c, a, attend_prefill_workspace(a), fixed, fixed_bytes, s));
            KV_HIP(launch_attend_prefill(a, s));
        }
        g_last_kernel = done ? 4 : 3;
    } else if (g_policy != 1 && attend_valu_supported(a)) {
        KV_TRY(bind_workspace(c, a, attend_valu_workspace(a), fixed, fixed_bytes, s));
        KV_HIP(launch_attend_valu(a, s));
        g_last_kernel = 5;
    } else {
        // a 16-bit quantized cache of head sizes above 256: dequantized into scratch pages, every call, for the
        // vector-ALU kernel (several times the bytes of a quantized decode kernel, a fiftieth of the plain kernel's time)
        bool done = false;
        if (!fixed && g_policy != 1 && attend_valu_dequant_first(a)) KV_TRY(attend_dequant_first(c, a, s, &done, true));
        g_last_kernel = done ? 6 : 0;
        if (!done) {
            KV_TRY(bind_workspace(c, a, attend_generic_workspace(a), fixed, fixed_bytes, s));
            KV_HIP(launch_attend_generic(a, s));
        }
    }
    if (user_out)
        KV_HIP(launch_repitch_rows(user_out, (size_t)c->Dv_user * c->st.es, out, (size_t)c->st.Dv * c->st.es, q_rows, s));
    return KVHIP_OK;
}
}  // namespace

kvhip_status kvhip_cache_attend(kvhip_cache *c, const void *q, int32_t B, int32_t Hq, int32_t L,
                                int32_t D, float scale, const kvhip_mask *mask, void *out, void *stream) {
    return attend_impl(c, q, B, Hq, L, D, scale, mask, out, stream, nullptr, 0);
}

kvhip_status kvhip_cache_attend_static(kvhip_cache *c, const void *q, int32_t B, int32_t Hq, int32_t L,
                                       int32_t D, float scale, const kvhip_mask *mask, void *out, void *stream) {
    int dev = -1;
    KV_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES || !g_scratch_ptr[dev])
        return fail(KVHIP_ERR_STATE, "kvhip_init has not run on the current device");
    return attend_impl(c, q, B, Hq, L, D, scale, mask, out, stream, g_scratch_ptr[dev], SCRATCH_BYTES);
}

kvhip_status kvhip_cache_update_attend(kvhip_cache *c, const void *q, const void *k, const void *v,
                                       int32_t B, int32_t Hq, int32_t Hkv, int32_t L, int32_t Dk,
                                       int32_t Dv, int32_t dtype, float scale, const kvhip_mask *mask,
                                       void *out, void *stream) {
    // One new token into a quantized cache: the decode kernel quantizes the row itself, so the
    // step is a single launch.  The bookkeeping of `updateQuantized` runs here as usual.
    if (c && k && v && q && out && L == 1 && c->kind == KVHIP_KIND_QUANTIZED && !c->staging && !c->rope &&
        (dtype == KVHIP_F16 || dtype == KVHIP_BF16) && (!mask || mask->mode == KVHIP_MASK_NONE) && c->has_geom &&
        c->has_buffers && !c->padded() && c->B == B && c->Hkv == Hkv && c->st.Dk == Dk && c->st.Dv == Dv && c->st.dtype == dtype) {
        KV_TRY(update_simple(c, k, v, 1, S(c, stream), false));
        const kvhip_status st = attend_impl(c, q, B, Hq, L, Dk, scale, mask, out, stream, nullptr, 0, k, v, (int32_t)c->offset - 1);
        if (st != KVHIP_OK) {  // nothing was written: take the row back
            c->offset -= 1;
            c->presented = c->offset;
        }
        return st;
    }
    // One new token into a full-precision cache of a 16-bit dtype (KVCacheSimple, or the in-place step of a
    // RotatingKVCache): the decode kernel copies the row into its slot itself.  The bookkeeping of `update`
    // runs here as usual; if the attention cannot be enqueued the row is written by the append kernel, so
    // the cache holds what its counters say.
    if (c && k && v && q && out && L == 1 && (c->kind == KVHIP_KIND_SIMPLE || c->kind == KVHIP_KIND_ROTATING) &&
        !c->staging && !c->rope && (dtype == KVHIP_F16 || dtype == KVHIP_BF16) && (!mask || mask->mode == KVHIP_MASK_NONE) &&
        c->has_geom && c->has_buffers && !c->padded() && c->B == B && c->Hkv == Hkv && c->st.Dk == Dk && c->st.Dv == Dv && c->st.dtype == dtype) {
        int32_t slot = -1;
        if (c->kind == KVHIP_KIND_SIMPLE) {
            KV_TRY(update_simple(c, k, v, 1, S(c, stream), false));
            slot = (int32_t)c->offset - 1;
        } else {
            KV_TRY(update_rotating(c, k, v, 1, S(c, stream), &slot));
        }
        const kvhip_status st = attend_impl(c, q, B, Hq, L, Dk, scale, mask, out, stream, nullptr, 0, k, v, slot);
        if (st != KVHIP_OK) (void)launch_append_fp(c->st, k, v, 1, 0, slot, 1, S(c, stream), nullptr);
        return st;
    }
    KV_TRY(kvhip_cache_update(c, k, v, B, Hkv, L, Dk, Dv, dtype, stream));
    return kvhip_cache_attend(c, q, B, Hq, L, Dk, scale, mask, out, stream);
}

kvhip_status kvhip_cache_mask_plan(const kvhip_cache *c, int32_t n, int32_t window, int32_t return_array,
                                   kvhip_mask_plan_t *p) {
    if (!c || !p) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    std::memset(p, 0, sizeof(*p));
    const bool has_w = window > 0;
    if (c->kind != KVHIP_KIND_ROTATING) {
        // BaseKVCache.makeMask, KVCache.swift:236-250
        if (n == 1) { p->mode = KVHIP_MASK_NONE; return KVHIP_OK; }
        if (return_array || (has_w && n > window)) {
            p->mode = KVHIP_MASK_ARRAY;
            p->rows = n;
            p->cols = (int32_t)c->offset + n;
            p->offset = (int32_t)c->offset;
            p->window = has_w ? window : 0;
            return KVHIP_OK;
        }
        p->mode = KVHIP_MASK_CAUSAL;
        return KVHIP_OK;
    }
    // RotatingKVCache.makeMask, KVCache.swift:834-871
    const int64_t M = c->max_size;
    if (n > 1) {
        const int64_t actual = has_w ? window : M;
        const int64_t capped = std::min(M - 1, c->offset);
        if (capped + n > actual || return_array) {
            p->mode = KVHIP_MASK_ARRAY;
            p->rows = n;
            p->cols = (int32_t)(capped + n);
            p->offset = (int32_t)capped;
            p->window = (int32_t)actual;
            return KVHIP_OK;
        }
        p->mode = KVHIP_MASK_CAUSAL;
        return KVHIP_OK;
    }
    if (!has_w) { p->mode = KVHIP_MASK_NONE; return KVHIP_OK; }
    if (c->offset >= window && M > window) {
        int64_t cur = c->idx;
        if (cur >= M) cur = 0;
        const int64_t size = c->offset < M ? c->offset + 1 : M;
        p->mode = KVHIP_MASK_ARRAY;
        p->rows = 1;
        p->cols = (int32_t)size;
        p->rolled = 1;
        p->roll_shift = (int32_t)(cur + 1);
        p->roll_window = window;
        return KVHIP_OK;
    }
    p->mode = KVHIP_MASK_NONE;
    return KVHIP_OK;
}

kvhip_status kvhip_mask_materialize(const kvhip_mask_plan_t *p, uint8_t *dst, void *stream) {
    if (!p || !dst) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (p->mode != KVHIP_MASK_ARRAY) return fail(KVHIP_ERR_INVALID_ARG, "plan does not describe an array mask");
    KV_HIP(launch_mask_materialize(*p, dst, S(stream)));
    return KVHIP_OK;
}

// ---- state -------------------------------------------------------------------
int32_t kvhip_cache_state_count(const kvhip_cache *c) {
    if (!c || !c->has_buffers) return 0;
    return c->kind == KVHIP_KIND_QUANTIZED ? 6 : 2;
}

kvhip_status kvhip_cache_state_desc(const kvhip_cache *c, int32_t i, int64_t shape[4], int32_t *dtype) {
    if (!c || !shape || !dtype) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (i < 0 || i >= kvhip_cache_state_count(c)) return fail(KVHIP_ERR_INVALID_ARG, "state index out of range");
    const Store &s = c->st;
    shape[0] = c->B;
    shape[1] = c->Hkv;
    shape[2] = state_rows(c);
    if (c->kind != KVHIP_KIND_QUANTIZED) {
        shape[3] = i == 0 ? c->Dk_user : c->Dv_user;
        *dtype = s.dtype;
        return KVHIP_OK;
    }
    const int D = i < 3 ? c->Dk_user : c->Dv_user;
    if (i % 3 == 0) {
        shape[3] = D * s.bits / 32;
        *dtype = KVHIP_U32;
    } else {
        shape[3] = D / s.gs;
        *dtype = s.dtype;
    }
    return KVHIP_OK;
}

kvhip_status kvhip_cache_state_export(const kvhip_cache *c, int32_t i, void *dst, void *stream) {
    if (!c) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (i < 0 || i >= kvhip_cache_state_count(c)) return fail(KVHIP_ERR_INVALID_ARG, "state index out of range");
    const int64_t n = state_rows(c);
    if (n == 0) return KVHIP_OK;  // (an array of no rows -- a cache trimmed back to empty -- has no address)
    if (!dst) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (c->kind == KVHIP_KIND_QUANTIZED) {
        if (!c->padded()) {
            KV_HIP(launch_export_quant(c->st, i, (int)n, dst, S(c, stream)));
            return KVHIP_OK;
        }
        // the array of the stored width first, then its leading columns (codes are a bit stream from column 0 on,
        // pairs come one per group: the caller's columns are a prefix of every row)
        const Store &st = c->st;
        const int Ds = i < 3 ? st.Dk : st.Dv, Du = i < 3 ? c->Dk_user : c->Dv_user;
        const size_t wide = i % 3 == 0 ? (size_t)Ds * st.bits / 8 : (size_t)(Ds / st.gs) * st.es;
        const size_t narrow = i % 3 == 0 ? (size_t)Du * st.bits / 8 : (size_t)(Du / st.gs) * st.es;
        const size_t rows = (size_t)st.BH * (size_t)n;
        void *tmp = nullptr;
        size_t got = 0;
        KV_HIP(pool_alloc(&tmp, rows * wide, &got));
        hipError_t e = launch_export_quant(st, i, (int)n, tmp, S(c, stream));
        if (e == hipSuccess) e = launch_repitch_rows(dst, narrow, tmp, wide, rows, S(c, stream));
        std::vector<std::pair<void *, size_t>> t{{tmp, got}};
        retire(std::move(t), S(c, stream));
        KV_HIP(e);
        return KVHIP_OK;
    }
    std::vector<int32_t> ident;
    const int32_t *slots = c->rows.data();
    if (c->kind != KVHIP_KIND_ROTATING) {
        ident.resize((size_t)n);
        for (size_t r = 0; r < ident.size(); ++r) ident[r] = (int32_t)r;
        slots = ident.data();
    }
    return export_slots(c, slots, n, i == 0 ? dst : nullptr, i == 1 ? dst : nullptr, S(c, stream));
}

kvhip_status kvhip_cache_state_import(kvhip_cache *c, int32_t count, const void *const *srcs,
                                      const int64_t *shapes, const int32_t *dtypes, void *stream) {
    if (!c || !srcs || !shapes || !dtypes) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (c->staging)  // RotatingStagedKVCache.swift:95-103
        return fail(KVHIP_ERR_STATE, "RotatingStagedKVCache is round-scoped and cannot be restored from state");
    const bool q = c->kind == KVHIP_KIND_QUANTIZED;
    if (q ? (count != 6) : (count != 2)) {
        if (q && count == 4) return fail(KVHIP_ERR_UNSUPPORTED, "quantized state without biases (non-affine mode) is not supported");
        return fail(KVHIP_ERR_STATE, q ? "QuantizedKVCache state must have exactly 6 or 4 arrays"
                                       : "cache state must have exactly 2 arrays (keys, values)");
    }
    const int64_t *k0 = shapes, *v0 = shapes + (q ? 12 : 4);
    const int64_t B = k0[0], H = k0[1], n = k0[2];
    for (int a = 0; a < count; ++a)
        if (shapes[4 * a] != B || shapes[4 * a + 1] != H || shapes[4 * a + 2] != n)
            return fail(KVHIP_ERR_INVALID_ARG, "state arrays disagree on batch, heads or rows");
    int Dk, Dv, dtype;
    if (q) {
        if (dtypes[0] != KVHIP_U32 || dtypes[3] != KVHIP_U32) return fail(KVHIP_ERR_INVALID_ARG, "packed codes must be uint32");
        Dk = (int)(k0[3] * 32 / c->bits);
        Dv = (int)(v0[3] * 32 / c->bits);
        dtype = dtypes[1];
        if (shapes[4 * 1 + 3] * c->gs != Dk || shapes[4 * 4 + 3] * c->gs != Dv)
            return fail(KVHIP_ERR_INVALID_ARG, "scales extent does not match head dim / group size");
    } else {
        Dk = (int)k0[3];
        Dv = (int)v0[3];
        dtype = dtypes[0];
    }
    {   // refuse a bad geometry before anything the cache holds is given up
        kvhip_cache probe;
        probe.kind = c->kind;
        probe.gs = c->gs;
        probe.bits = c->bits;
        KV_TRY(set_geometry(&probe, (int)B, (int)H, Dk, Dv, dtype));
    }
    // a state setter replaces the buffers wholesale (the old pages go once the work enqueued
    // on this stream so far, which may still read them, has run)
    drop_pages(c, S(c, stream), false);
    c->st = Store();
    c->has_geom = false;
    c->rows.clear();
    c->used.clear();
    c->cursor = 0;
    KV_TRY(set_geometry(c, (int)B, (int)H, Dk, Dv, dtype));
    hipStream_t s = S(c, stream);
    KV_TRY(ensure_slots(c, std::max<int64_t>(n, 1), s, true));
    const void *wide_srcs[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    std::vector<std::pair<void *, size_t>> tmp;
    if (c->padded() && n > 0) {
        // arrays of the stored widths, the added columns zero (codes 0 with scale 0 and bias 0 are zero values)
        const Store &st = c->st;
        const size_t rows = (size_t)st.BH * (size_t)n;
        hipError_t e = hipSuccess;
        for (int a = 0; a < count && e == hipSuccess; ++a) {
            const bool keys = q ? a < 3 : a == 0;
            const int Ds = keys ? st.Dk : st.Dv, Du = keys ? c->Dk_user : c->Dv_user;
            const size_t wide = !q ? (size_t)Ds * st.es : (a % 3 == 0 ? (size_t)Ds * st.bits / 8 : (size_t)(Ds / st.gs) * st.es);
            const size_t narrow = !q ? (size_t)Du * st.es : (a % 3 == 0 ? (size_t)Du * st.bits / 8 : (size_t)(Du / st.gs) * st.es);
            void *p = nullptr;
            size_t got = 0;
            e = pool_alloc(&p, rows * wide, &got);
            if (e != hipSuccess) break;
            tmp.push_back({p, got});
            e = launch_repitch_rows(p, wide, srcs[a], narrow, rows, s);
            wide_srcs[a] = p;
        }
        if (e != hipSuccess) {
            retire(std::move(tmp), s);
            KV_HIP(e);
        }
        srcs = wide_srcs;
    }
    {
        const hipError_t e = q ? launch_import_quant(c->st, srcs, (int)n, s) : launch_import_fp(c->st, srcs[0], srcs[1], (int)n, s);
        retire(std::move(tmp), s);
        KV_HIP(e);
    }
    c->has_buffers = true;
    c->ref_len = n;
    c->presented = n;
    if (c->kind == KVHIP_KIND_SIMPLE) c->offset = n;  // KVCache.swift:467
    if (c->kind == KVHIP_KIND_ROTATING) {
        c->rows.resize((size_t)n);
        for (int64_t r = 0; r < n; ++r) {
            c->rows[(size_t)r] = (int32_t)r;
            c->used[(size_t)r] = 1;
        }
        c->cursor = n;
    }
    return KVHIP_OK;
}

int32_t kvhip_cache_meta_count(const kvhip_cache *c) {
    if (!c) return 0;
    return c->kind == KVHIP_KIND_SIMPLE ? 1 : (c->kind == KVHIP_KIND_ROTATING ? 6 : 4);
}

int32_t kvhip_cache_meta_get(const kvhip_cache *c, int32_t i, char *buf, int32_t len) {
    if (!c || !buf || len <= 0) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (i < 0 || i >= kvhip_cache_meta_count(c)) return fail(KVHIP_ERR_INVALID_ARG, "meta index out of range");
    std::string v;
    if (c->kind == KVHIP_KIND_ROTATING) {
        const int64_t vals[5] = {c->keep, c->max_size, c->step, c->offset, c->idx};
        v = i < 5 ? std::to_string(vals[i]) : c->origin;
    } else if (c->kind == KVHIP_KIND_QUANTIZED) {
        const int64_t vals[4] = {c->step, c->offset, c->gs, c->bits};
        v = std::to_string(vals[i]);
    }
    if ((int32_t)v.size() + 1 > len) return fail(KVHIP_ERR_INVALID_ARG, "buffer too small");
    std::memcpy(buf, v.c_str(), v.size() + 1);
    return (int32_t)v.size();
}

static bool parse_int(const char *s, int64_t &out) {
    if (!s || !*s) return false;
    char *end = nullptr;
    const long long v = std::strtoll(s, &end, 10);
    if (*end) return false;
    out = v;
    return true;
}

kvhip_status kvhip_cache_meta_set(kvhip_cache *c, int32_t count, const char *const *values) {
    if (!c || !values) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (c->staging)  // RotatingStagedKVCache.swift:105-111
        return fail(KVHIP_ERR_STATE, "RotatingStagedKVCache is round-scoped and cannot be restored from metaState");
    if (c->kind == KVHIP_KIND_SIMPLE) {
        if (count != 1 || !values[0] || values[0][0])
            return fail(KVHIP_ERR_STATE, "This cache has no meta_state but a meta_state was set.");
        return KVHIP_OK;
    }
    if (c->kind == KVHIP_KIND_ROTATING) {
        // KVCache.swift:782-815
        if (count != 5 && count != 6) return fail(KVHIP_ERR_STATE, "RotatingKVCache metaState must have 5 or 6 values");
        int64_t keep, step, off, idx, mx;
        if (!parse_int(values[0], keep) || !parse_int(values[2], step) || !parse_int(values[3], off) || !parse_int(values[4], idx))
            return fail(KVHIP_ERR_STATE, "Failed to convert metaState values to integers");
        if (values[1] && std::strcmp(values[1], "None") == 0)
            return fail(KVHIP_ERR_STATE, "RotatingKVCache requires a non-nil maxSize. Cannot load cache with maxSize=None.");
        if (!parse_int(values[1], mx)) return fail(KVHIP_ERR_STATE, "Failed to convert maxCacheSize to integer");
        std::string origin = "modelNative";
        if (count == 6) {
            origin = values[5] ? values[5] : "";
            if (origin != "modelNative" && origin != "requested")
                return fail(KVHIP_ERR_STATE, "Invalid RotatingKVCache capacity origin '" + origin + "'");
        }
        c->keep = keep;
        c->max_size = mx;
        c->step = (int)step;
        c->offset = off;
        c->idx = idx;
        c->origin = origin;
        return KVHIP_OK;
    }
    // KVCache.swift:1148-1166
    if (count != 4) return fail(KVHIP_ERR_STATE, "QuantizedKVCache metaState must have exactly 4 values");
    int64_t off, gs, bits;
    if (!parse_int(values[1], off) || !parse_int(values[2], gs) || !parse_int(values[3], bits))
        return fail(KVHIP_ERR_STATE, "Failed to convert QuantizedKVCache metaState values to integers");
    if (c->has_geom && c->cap_pages > 0 && (gs != c->gs || bits != c->bits))
        return fail(KVHIP_ERR_UNSUPPORTED, "group size / bits differ from the arrays this cache already holds");
    c->offset = off;
    c->gs = (int)gs;
    c->bits = (int)bits;
    return KVHIP_OK;
}

// ---- copy / views / conversions -------------------------------------------------
kvhip_status kvhip_cache_copy(const kvhip_cache *c, void *stream, kvhip_cache **out) {
    if (!c || !out) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (c->staging)  // RotatingStagedKVCache.swift:123-125
        return fail(KVHIP_ERR_STATE, "RotatingStagedKVCache is round-scoped and cannot be copied");
    hipStream_t s = S(c, stream);
    kvhip_cache *n = new_cache_like(c);
    const int64_t rows = state_rows(c);
    if (c->has_buffers) {
        // `new.state = self.state`: the copy's buffers hold exactly the exported rows
        n->has_geom = false;
        kvhip_status st = set_geometry(n, c->B, c->Hkv, c->Dk_user, c->Dv_user, c->st.dtype);
        if (st == KVHIP_OK) st = ensure_slots(n, std::max<int64_t>(rows, 1), s, true);
        if (st != KVHIP_OK) { kvhip_cache_free(n); return st; }
        if (c->kind == KVHIP_KIND_QUANTIZED) {
            const int64_t pages = (rows + PAGE - 1) / PAGE;
            KV_HIP_OR(launch_copy_pages(c->st, n->st, (int)pages, s), kvhip_cache_free(n));
        } else {
            std::vector<int32_t> ident;
            const int32_t *slots = c->rows.data();
            if (c->kind != KVHIP_KIND_ROTATING) {
                ident.resize((size_t)rows);
                for (size_t r = 0; r < ident.size(); ++r) ident[r] = (int32_t)r;
                slots = ident.data();
            }
            const RunList rl = runs_of(slots, rows);
            for (size_t first = 0; first < rl.size(); first += MAXRUNS) {
                const size_t cnt = std::min((size_t)MAXRUNS, rl.size() - first);
                KV_HIP_OR(launch_compact_fp(c->st, pack_runs(rl, first, cnt), n->st, (int)rows, s), kvhip_cache_free(n));
            }
        }
        n->has_buffers = true;
        n->ref_len = rows;
        n->presented = rows;
        (void)S(n, stream);
        if (c->kind == KVHIP_KIND_ROTATING) {
            n->rows.resize((size_t)rows);
            for (int64_t r = 0; r < rows; ++r) {
                n->rows[(size_t)r] = (int32_t)r;
                n->used[(size_t)r] = 1;
            }
            n->cursor = rows;
        }
    }
    if (c->kind == KVHIP_KIND_SIMPLE) n->offset = c->has_buffers ? rows : 0;  // copy goes through state only
    else {
        n->offset = c->offset;
        n->idx = c->idx;
        n->origin = c->origin;
    }
    *out = n;
    return KVHIP_OK;
}

// ---- staged rounds on a ring (RotatingStagedKVCache.swift, KVCacheRound.swift:128-156) ------
kvhip_status kvhip_cache_stage_begin(kvhip_cache *c) {
    if (!c) return fail(KVHIP_ERR_INVALID_ARG, "null cache");
    if (c->kind != KVHIP_KIND_ROTATING)
        return fail(KVHIP_ERR_INVALID_ARG, "only RotatingKVCache stages a round; append-only caches are written through and trimmed");
    if (c->staging) return fail(KVHIP_ERR_STATE, "a staged round is already open on this cache");
    c->staging = true;
    c->staged.clear();
    c->stage_view.clear();
    c->presented_live = c->presented;
    return KVHIP_OK;
}

int32_t kvhip_cache_stage_is_open(const kvhip_cache *c) { return c && c->staging; }

int64_t kvhip_cache_stage_count(const kvhip_cache *c) { return c ? (int64_t)c->staged.size() : -1; }

kvhip_status kvhip_cache_stage_fetch(const kvhip_cache *c, void *dk, void *dv, void *stream) {
    if (!c) return fail(KVHIP_ERR_INVALID_ARG, "null cache");
    if (!c->staging || c->staged.empty()) return fail(KVHIP_ERR_STATE, "nothing is staged");
    return export_slots(c, c->staged.data(), (int64_t)c->staged.size(), dk, dv, S(c, stream));
}

kvhip_status kvhip_cache_stage_commit(kvhip_cache *c, int64_t retaining, void *stream) {
    if (!c) return fail(KVHIP_ERR_INVALID_ARG, "null cache");
    if (!c->staging) return fail(KVHIP_ERR_STATE, "no staged round is open on this cache");
    hipStream_t s = S(c, stream);
    // RotatingStagedKVCache.swift:62-76: the first `keep` staged rows go to the ring through
    // the normal write path, the rest are dropped.  The kept rows are first gathered into a
    // dense pair (a few rows), because the normal write path may reuse their slots.
    const int64_t keep = std::min<int64_t>(std::max<int64_t>(retaining, 0), (int64_t)c->staged.size());
    kvhip_status st = KVHIP_OK;
    if (keep > 0) {
        if ((size_t)keep > c->stage_tmp_rows) {
            // a larger pair replaces the old one, which an earlier commit's append may still read:
            // it stays allocated until the cache is freed (no wait for the device here)
            if (c->stage_tmp_k) c->parked.push_back({c->stage_tmp_k, (size_t)0});
            if (c->stage_tmp_v) c->parked.push_back({c->stage_tmp_v, (size_t)0});
            c->stage_tmp_k = c->stage_tmp_v = nullptr;
            c->stage_tmp_rows = 0;
            const size_t rows = (size_t)std::max<int64_t>(2 * keep, 16);
            KV_HIP(hipMalloc(&c->stage_tmp_k, (size_t)c->st.BH * rows * c->st.Dk * c->st.es));
            KV_HIP(hipMalloc(&c->stage_tmp_v, (size_t)c->st.BH * rows * c->st.Dv * c->st.es));
            c->stage_tmp_rows = rows;
        }
        st = export_slots_stored(c, c->staged.data(), keep, c->stage_tmp_k, c->stage_tmp_v, s);
    }
    for (int32_t slot : c->staged) c->used[(size_t)slot] = 0;
    c->staged.clear();
    c->stage_view.clear();
    c->staging = false;
    c->presented = c->presented_live;
    if (st != KVHIP_OK) return st;
    if (keep > 0) return update_rotating(c, c->stage_tmp_k, c->stage_tmp_v, (int)keep, s);
    return KVHIP_OK;
}

kvhip_status kvhip_cache_logical_view(const kvhip_cache *c, int64_t tail, int64_t *out_rows, void *dk,
                                      void *dv, void *stream) {
    if (!c || !out_rows) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (c->kind != KVHIP_KIND_ROTATING) return fail(KVHIP_ERR_INVALID_ARG, "logicalView belongs to RotatingKVCache");
    if (!c->has_buffers) return fail(KVHIP_ERR_STATE, "logicalView before the first write");
    const std::vector<int32_t> ordered = logical_rows(c, tail);
    *out_rows = (int64_t)ordered.size();
    if ((dk || dv) && !ordered.empty())
        return export_slots(c, ordered.data(), (int64_t)ordered.size(), dk, dv, S(c, stream));
    return KVHIP_OK;
}

kvhip_status kvhip_cache_to_quantized(const kvhip_cache *c, int32_t group_size, int32_t bits, void *stream,
                                      kvhip_cache **out) {
    if (!c || !out) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (c->kind == KVHIP_KIND_ROTATING)
        return fail(KVHIP_ERR_STATE,
                    "RotatingKVCache quantization is not implemented because its temporal ordering requires dedicated handling.");
    if (c->kind != KVHIP_KIND_SIMPLE) return fail(KVHIP_ERR_INVALID_ARG, "toQuantized belongs to KVCacheSimple");
    if (group_size <= 0) group_size = 64;
    if (bits <= 0) bits = 4;
    hipStream_t s = S(c, stream);
    kvhip_config cfg{KVHIP_KIND_QUANTIZED, 0, 0, 0, group_size, bits};
    if (!c->has_buffers) {
        KV_TRY(kvhip_cache_create(&cfg, out));
        (*out)->offset = c->offset;
        return KVHIP_OK;
    }
    const int eff = kvhip_resolved_group_size(group_size, c->Dk_user, c->Dv_user);
    if (!eff)
        return fail(KVHIP_ERR_STATE,
                    "KV cache quantization requires head dimensions divisible by one of the supported group sizes (32, 64, 128).");
    cfg.group_size = eff;
    kvhip_cache *n = nullptr;
    KV_TRY(kvhip_cache_create(&cfg, &n));
    const int64_t rows = std::max<int64_t>(c->offset, 0);
    kvhip_status st = set_geometry(n, c->B, c->Hkv, c->Dk_user, c->Dv_user, c->st.dtype);
    // (the conversion goes from pages to pages: both caches have to store the same head sizes)
    if (st == KVHIP_OK && (n->st.Dk != c->st.Dk || n->st.Dv != c->st.Dv))
        st = fail(KVHIP_ERR_UNSUPPORTED, "a quantized cache of this group size stores other head sizes than the cache being converted");
    if (st == KVHIP_OK) st = ensure_slots(n, std::max<int64_t>(rows, 1), s, true);
    if (st != KVHIP_OK) { kvhip_cache_free(n); return st; }
    // one pass from the full-precision pages into the new cache's pages, enqueued on the stream
    const int64_t have = std::min(rows, c->cap_slots());  // (an offset set past the buffers has no rows behind it)
    if (have > 0) KV_HIP_OR(launch_requant_pages(c->st, n->st, (int)have, s), kvhip_cache_free(n));
    (void)S(n, stream);
    n->has_buffers = true;
    n->ref_len = rows;  // the state setter keeps the arrays' extent
    n->presented = rows;
    n->offset = c->offset;
    *out = n;
    return KVHIP_OK;
}

kvhip_status kvhip_cache_to_unquantized(const kvhip_cache *c, void *stream, kvhip_cache **out) {
    if (!c || !out) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (c->kind != KVHIP_KIND_QUANTIZED) return fail(KVHIP_ERR_INVALID_ARG, "toUnquantized belongs to QuantizedKVCache");
    hipStream_t s = S(c, stream);
    kvhip_config cfg{KVHIP_KIND_SIMPLE, 0, 0, 0, 0, 0};
    kvhip_cache *n = nullptr;
    KV_TRY(kvhip_cache_create(&cfg, &n));
    n->offset = c->offset;
    if (!c->has_buffers) { *out = n; return KVHIP_OK; }
    const int64_t rows = std::max<int64_t>(std::min(c->offset, c->ref_len), 0);
    const Store &q = c->st;
    kvhip_status st = set_geometry(n, c->B, c->Hkv, c->Dk_user, c->Dv_user, q.dtype);
    if (st == KVHIP_OK && (n->st.Dk != q.Dk || n->st.Dv != q.Dv))
        st = fail(KVHIP_ERR_UNSUPPORTED, "a full-precision cache stores other head sizes than the quantized cache being converted");
    if (st == KVHIP_OK) st = ensure_slots(n, std::max<int64_t>(rows, 1), s, true);
    if (st != KVHIP_OK) { kvhip_cache_free(n); return st; }
    if (rows > 0) KV_HIP_OR(launch_dequant_pages(q, n->st, (int)rows, s), kvhip_cache_free(n));
    (void)S(n, stream);
    n->has_buffers = true;
    n->ref_len = rows;
    n->presented = rows;
    n->offset = rows;  // `simpleCache.state = ...` sets offset to the arrays' extent
    *out = n;
    return KVHIP_OK;
}

kvhip_status kvhip_affine_quantize(const void *src, int64_t rows, int32_t D, int32_t gs, int32_t bits,
                                   int32_t dtype, uint32_t *wq, void *scales, void *biases, void *stream) {
    if (!src || !wq || !scales || !biases) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (!affine_bits_ok(bits)) return fail(KVHIP_ERR_UNSUPPORTED, "bits must be 2, 3, 4, 5, 6 or 8");
    if ((gs != 32 && gs != 64 && gs != 128) || D % gs) return fail(KVHIP_ERR_INVALID_ARG, "group size must be 32, 64 or 128 and divide D");
    if (dtype < 0 || dtype > 2) return fail(KVHIP_ERR_INVALID_ARG, "bad dtype");
    KV_HIP(launch_affine_quantize(src, rows, D, gs, bits, dtype, wq, scales, biases, S(stream)));
    return KVHIP_OK;
}

kvhip_status kvhip_affine_dequantize(const uint32_t *wq, const void *scales, const void *biases,
                                     int64_t rows, int32_t D, int32_t gs, int32_t bits, int32_t dtype,
                                     void *dst, void *stream) {
    if (!wq || !scales || !biases || !dst) return fail(KVHIP_ERR_INVALID_ARG, "null argument");
    if (!affine_bits_ok(bits)) return fail(KVHIP_ERR_UNSUPPORTED, "bits must be 2, 3, 4, 5, 6 or 8");
    if (D % gs) return fail(KVHIP_ERR_INVALID_ARG, "group size must divide D");
    if (dtype < 0 || dtype > 2) return fail(KVHIP_ERR_INVALID_ARG, "bad dtype");
    KV_HIP(launch_affine_dequantize(wq, scales, biases, rows, D, gs, bits, dtype, dst, S(stream)));
    return KVHIP_OK;
}

}  // extern "C"
