// Host side of libtract_rocm.so: the C ABI declared in include/tract_rocm.h.
// Runtime context, error convention, device memory, the in-place capacity-doubling KV
// cache and the dispatch of attention calls to the kernels.
#include <atomic>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <iterator>
#include <map>
#include <mutex>
#include <new>
#include <vector>
#include "common.h"

namespace trocm {

// ---- error convention (api/ffi/src/lib.rs:18-62) -----------------------------------------
static thread_local char g_last_error[1024] = "";

int fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return 1;
}

// ---- context ---------------------------------------------------------------------------------
static std::mutex g_init_mutex;
static std::atomic<int> g_device{-1};   // written once, under g_init_mutex; read by every call
static int g_compute_units = 0;
static size_t g_hbm_bytes = 0;
static char g_name[256] = "";

// Split-K scratch of trocm_sdpa_cached_noalloc, the entry point that allocates nothing: the workspace its
// kernels would otherwise take from the caller.  The array's name is a host-side stand-in, not a device
// address; trocm_init asks the runtime where the array lives on the library's device, and every use on the
// host goes through that pointer.  All calls share the one array: calls that overlap in time race on it.
static __device__ __align__(256) unsigned char scratch[TROCM_STATIC_SCRATCH_BYTES];
static void *g_scratch_ptr = nullptr;   // written once, under g_init_mutex, before g_device is published

struct ThreadStream {
    hipStream_t s = nullptr;
    ~ThreadStream() {
        // Streams of exiting threads are left to the runtime: destroying them here can run
        // after the HIP runtime itself has been torn down.
    }
};
static thread_local ThreadStream g_thread_stream;

int ensure_init() {
    if (g_device >= 0) return 0;
    return fail("trocm_init() has not been called");
}

int num_compute_units() { return g_compute_units > 0 ? g_compute_units : 256; }

int resolve_stream(void *stream, hipStream_t *out) {
    if (ensure_init()) return 1;
    if (stream) {
        *out = (hipStream_t)stream;
        return 0;
    }
    if (!g_thread_stream.s) {
        TROCM_HIP(hipSetDevice(g_device));
        TROCM_HIP(hipStreamCreateWithFlags(&g_thread_stream.s, hipStreamNonBlocking));
    }
    *out = g_thread_stream.s;
    return 0;
}

}  // namespace trocm

using namespace trocm;

// ---- KV pool: one device allocation carved into per-cache planes ------------------------------
// (the role of DeviceMemoryPool, gpu/src/memory/pool.rs, for state that outlives a run).
// Address-ordered first fit with coalescing; 256-byte granularity; guarded by a mutex.
struct trocm_kv_pool {
    char *base = nullptr;
    size_t bytes = 0, in_use = 0;
    int64_t live_caches = 0;
    std::map<size_t, size_t> free_list;  // offset -> size
    std::map<size_t, size_t> used;       // offset -> size
    std::mutex mu;
};

static void *pool_alloc(trocm_kv_pool *pool, size_t bytes) {
    bytes = (bytes + 255) & ~(size_t)255;
    if (bytes == 0) bytes = 256;
    std::lock_guard<std::mutex> lock(pool->mu);
    for (auto it = pool->free_list.begin(); it != pool->free_list.end(); ++it) {
        if (it->second >= bytes) {
            size_t off = it->first, rest = it->second - bytes;
            pool->free_list.erase(it);
            if (rest) pool->free_list[off + bytes] = rest;
            pool->used[off] = bytes;
            pool->in_use += bytes;
            return pool->base + off;
        }
    }
    return nullptr;
}

static void pool_free(trocm_kv_pool *pool, void *ptr) {
    std::lock_guard<std::mutex> lock(pool->mu);
    size_t off = (size_t)((char *)ptr - pool->base);
    auto u = pool->used.find(off);
    if (u == pool->used.end()) return;
    size_t size = u->second;
    pool->used.erase(u);
    pool->in_use -= size;
    auto next = pool->free_list.lower_bound(off);
    if (next != pool->free_list.end() && off + size == next->first) {  // merge with the block after
        size += next->second;
        next = pool->free_list.erase(next);
    }
    if (next != pool->free_list.begin()) {  // merge with the block before
        auto prev = std::prev(next);
        if (prev->first + prev->second == off) {
            prev->second += size;
            return;
        }
    }
    pool->free_list[off] = size;
}

// ---- KV cache object -------------------------------------------------------------------------
struct trocm_kv_cache {
    int fmt;
    int64_t B, H, D;
    int64_t len, cap, reallocs;
    int64_t pitch;  // tokens between the rows of consecutive heads in the planes (>= cap, see pitch_for)
    void *data;    // F32/F16 rows, or the code plane
    void *scales;  // f16 scale plane of the quantised formats
    trocm_kv_pool *pool;  // where the planes live; NULL = their own hipMalloc
    // sliding-window (ring buffer) mode, window_kv_cache.rs:80-87: capacity fixed at `window`,
    // `cursor` = next write position; 0 = ordinary growing cache
    int64_t window, cursor;
};

// Planes that a growing cache has left behind.  Work queued on the stream may still read them, so they are not
// freed at once (that would take a stream synchronisation inside an asynchronous append): an event recorded on the
// stream after the copy into the new planes guards them, and they are released by a later call that finds the
// event complete (growth, reserve, destroy, pool statistics), or that needs the memory and waits for it.
struct DeferredFree {
    void *data, *scales;
    trocm_kv_pool *pool;   // NULL: planes of their own (hipFree)
    hipEvent_t done;
};
static std::mutex g_deferred_mu;
static std::vector<DeferredFree> g_deferred;

static void release_planes(trocm_kv_pool *pool, void *data, void *scales) {
    if (pool) {
        if (data) pool_free(pool, data);
        if (scales) pool_free(pool, scales);
    } else {
        if (data) (void)hipFree(data);
        if (scales) (void)hipFree(scales);
    }
}

// Release the deferred planes whose event has completed; with `wait`, all of them (of `only_pool`, if given).
// hipFree waits for the whole device, so planes outside a pool are released only where the host is waiting anyway
// (`unpooled`: the synchronising calls, destroy, a failed allocation, trocm_release_unused); a pool's bookkeeping
// costs nothing.  The list's lock is not held while an event is waited for.
static void reap_deferred(bool wait, trocm_kv_pool *only_pool = nullptr, bool unpooled = true) {
    std::vector<DeferredFree> mine, ready;
    {
        std::lock_guard<std::mutex> lock(g_deferred_mu);
        for (size_t i = 0; i < g_deferred.size();) {
            const DeferredFree &d = g_deferred[i];
            if ((only_pool == nullptr || d.pool == only_pool) && (unpooled || d.pool != nullptr)) {
                mine.push_back(d);
                g_deferred[i] = g_deferred.back();
                g_deferred.pop_back();
            } else {
                i++;
            }
        }
    }
    std::vector<DeferredFree> pending;
    for (DeferredFree &d : mine) {
        bool done = hipEventQuery(d.done) == hipSuccess;
        if (!done && wait) done = hipEventSynchronize(d.done) == hipSuccess;
        (done ? ready : pending).push_back(d);
    }
    (void)hipGetLastError();   // "not ready" is an answer, not a failure: keep it away from the launch checks
    if (!pending.empty()) {
        std::lock_guard<std::mutex> lock(g_deferred_mu);
        g_deferred.insert(g_deferred.end(), pending.begin(), pending.end());
    }
    for (DeferredFree &d : ready) {
        (void)hipEventDestroy(d.done);
        release_planes(d.pool, d.data, d.scales);
    }
}

// Hand the planes over to the deferred list, guarded by an event recorded on `s` now.
static int defer_free(trocm_kv_pool *pool, void *data, void *scales, hipStream_t s) {
    if (!data && !scales) return 0;
    DeferredFree d{data, scales, pool, nullptr};
    hipError_t e = hipEventCreateWithFlags(&d.done, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventRecord(d.done, s);
    if (e != hipSuccess) {   // no event: fall back to waiting for the stream
        if (d.done) (void)hipEventDestroy(d.done);
        TROCM_HIP(hipStreamSynchronize(s));
        release_planes(pool, data, scales);
        return 0;
    }
    std::lock_guard<std::mutex> lock(g_deferred_mu);
    g_deferred.push_back(d);
    return 0;
}

// The same service for the other stateful objects of the library (the affine-quantised stores): device memory that
// work queued on `s` may still read is released by a later call, not by waiting for the stream here.
namespace trocm {
int defer_device_free(void *a, void *b, hipStream_t s) { return defer_free(nullptr, a, b, s); }
void reap_device_frees(bool wait) { reap_deferred(wait); }
}  // namespace trocm

static int plane_alloc(trocm_kv_cache *c, void **ptr, size_t bytes, const char *what) {
    if (c->pool) {
        *ptr = pool_alloc(c->pool, bytes);
        if (!*ptr) {   // planes of this pool that wait for their event may make the room
            reap_deferred(true, c->pool);
            *ptr = pool_alloc(c->pool, bytes);
        }
        if (!*ptr) {
            std::lock_guard<std::mutex> lock(c->pool->mu);
            return fail("KV pool exhausted: %s of %zu bytes does not fit (%zu of %zu bytes in use)", what, bytes,
                        c->pool->in_use, c->pool->bytes);
        }
        return 0;
    }
    hipError_t e = hipMalloc(ptr, bytes ? bytes : 16);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        reap_deferred(true);
        e = hipMalloc(ptr, bytes ? bytes : 16);
    }
    if (e != hipSuccess) return fail("allocating %s (%zu bytes) failed: %s", what, bytes, hipGetErrorString(e));
    return 0;
}

static int plane_free(trocm_kv_cache *c, void *ptr) {
    if (!ptr) return 0;
    if (c->pool) {
        pool_free(c->pool, ptr);
        return 0;
    }
    TROCM_HIP(hipFree(ptr));
    return 0;
}

// Row pitch (tokens between the rows of consecutive (batch, head) pairs) for a capacity.
// Capacities double, so `cap * row_bytes` is a large power of two for the usual head sizes, and a
// cache that is half full (the state right after a doubling) then leaves one address bit constant
// over the whole working set: measured on MI355X, decode over such a layout is 7 % slower than
// over densely packed rows (57.5 us against 53.5 us, batch 8, 8226 tokens in 16384-token rows).
// 1/32 of padding per row removes the effect (52.9 us).  TROCM_KV_PITCH_PAD=<tokens> overrides.
static int64_t pitch_for(int64_t cap) {
    static const int64_t forced = getenv("TROCM_KV_PITCH_PAD") ? atoll(getenv("TROCM_KV_PITCH_PAD")) : -1;
    if (forced >= 0) return cap + forced;
    return cap >= 2048 ? cap + ((cap / 32 + 7) & ~(int64_t)7) : cap;
}

static size_t plane_bytes(const trocm_kv_cache *c, int64_t cap) {
    return (size_t)c->B * c->H * cap * device_row_bytes(c->fmt, c->D);
}
static size_t scale_plane_bytes(const trocm_kv_cache *c, int64_t cap) {
    return is_quant(c->fmt) ? (size_t)c->B * c->H * cap * (c->D / 32) * 2 : 0;
}

// Copy the first `len` tokens of planes with capacity `src_cap` into planes of `dst_cap`.
static int copy_valid(const trocm_kv_cache *c, void *dst, void *dst_scales, int64_t dst_cap, const void *src,
                      const void *src_scales, int64_t src_cap, int64_t len, hipStream_t s) {
    if (len == 0) return 0;
    CopyNd d;
    d.rank = 2;
    int64_t rb = (int64_t)device_row_bytes(c->fmt, c->D);
    d.shape[0] = c->B * c->H;
    d.shape[1] = len * rb;
    d.dst_stride[0] = dst_cap * rb;
    d.src_stride[0] = src_cap * rb;
    d.dst_stride[1] = d.src_stride[1] = 1;
    if (launch_copy_nd(dst, src, d, 1, s)) return 1;
    if (is_quant(c->fmt)) {
        int64_t sb = c->D / 32 * 2;
        d.shape[1] = len * sb;
        d.dst_stride[0] = dst_cap * sb;
        d.src_stride[0] = src_cap * sb;
        if (launch_copy_nd(dst_scales, src_scales, d, 1, s)) return 1;
    }
    return 0;
}

// Replace the buffers by ones of `new_cap` tokens holding the valid region
// (grow(), transformers/src/ops/inplace_kv_cache.rs:106-113; the tail stays uninitialised).
static int regrow(trocm_kv_cache *c, int64_t new_cap, hipStream_t s) {
    reap_deferred(false, nullptr, false);
    void *nd = nullptr, *ns = nullptr;
    const int64_t new_pitch = pitch_for(new_cap);
    size_t pb = plane_bytes(c, new_pitch), sb = scale_plane_bytes(c, new_pitch);
    if (plane_alloc(c, &nd, pb, "a KV cache plane")) return 1;
    if (sb && plane_alloc(c, &ns, sb, "a KV cache scale plane")) {
        (void)plane_free(c, nd);
        return 1;
    }
    if (c->data && c->len) {
        if (copy_valid(c, nd, ns, new_pitch, c->data, c->scales, c->pitch, c->len, s)) {
            (void)plane_free(c, nd);
            (void)plane_free(c, ns);
            return 1;
        }
    }
    // The old planes may still be read by work queued on the stream (the copy above, earlier attention calls):
    // they are released once an event recorded here has completed, by a later call; the host does not wait.
    if (c->data && defer_free(c->pool, c->data, c->scales, s)) {
        (void)plane_free(c, nd);
        (void)plane_free(c, ns);
        return 1;
    }
    c->data = nd;
    c->scales = ns;
    c->cap = new_cap;
    c->pitch = new_pitch;
    return 0;
}

// A call that grew K and then failed to grow V (a pool that ran out) leaves the two capacities apart, and attention
// takes one row pitch for both: the next call brings the smaller cache up to the larger before anything else.
static int equalise_capacities(trocm_kv_cache *kc, trocm_kv_cache *vc, hipStream_t s) {
    if (kc->cap == vc->cap || kc->window || vc->window) return 0;
    trocm_kv_cache *small = kc->cap < vc->cap ? kc : vc, *big = kc->cap < vc->cap ? vc : kc;
    if (regrow(small, big->cap, s)) return 1;
    small->reallocs += 1;   // the growth that the failed call owed
    return 0;
}

extern "C" {

// ---- runtime -------------------------------------------------------------------------------
int trocm_init(int device) {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_device >= 0) {
        TROCM_REQUIRE(g_device.load() == device, "Context is already set on device %d", g_device.load());  // gpu/src/device.rs:129-137
        return 0;
    }
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n == 0)
        return fail("no HIP device available (%s)", e != hipSuccess ? hipGetErrorString(e) : "device count is 0");
    TROCM_REQUIRE(device >= 0 && device < n, "device %d out of range (found %d)", device, n);
    TROCM_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    TROCM_HIP(hipGetDeviceProperties(&prop, device));
    TROCM_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0,
                  "this library is built for gfx950 (MI355X); device %d is %s", device, prop.gcnArchName);
    g_compute_units = prop.multiProcessorCount;
    g_hbm_bytes = prop.totalGlobalMem;
    snprintf(g_name, sizeof(g_name), "%s (%s)", prop.name, prop.gcnArchName);
    // The device address of the static scratch on this device, and its counter area cleared once: the
    // kernels leave the counters at zero after every launch.
    void *sp = nullptr;
    TROCM_HIP(hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)));
    TROCM_REQUIRE(sp != nullptr, "hipGetSymbolAddress returned no address for the static scratch");
    TROCM_HIP(hipMemset(sp, 0, kWsCounterBytes));
    TROCM_HIP(hipDeviceSynchronize());
    g_scratch_ptr = sp;
    g_device = device;
    return 0;
}

const char *trocm_last_error(void) { return g_last_error; }

int trocm_device_info(int *compute_units, size_t *hbm_bytes, char *name, size_t name_len) {
    if (ensure_init()) return 1;
    if (compute_units) *compute_units = g_compute_units;
    if (hbm_bytes) *hbm_bytes = g_hbm_bytes;
    if (name && name_len) snprintf(name, name_len, "%s", g_name);
    return 0;
}

// ---- memory and streams ----------------------------------------------------------------------
int trocm_malloc(void **ptr, size_t bytes) {
    TROCM_NOT_NULL(ptr);
    if (ensure_init()) return 1;
    *ptr = nullptr;
    hipError_t e = hipMalloc(ptr, bytes ? bytes : 16);
    if (e != hipSuccess) return fail("device allocation of %zu bytes failed: %s", bytes, hipGetErrorString(e));
    return 0;
}

int trocm_free(void *ptr) {
    if (!ptr) return 0;
    TROCM_HIP(hipFree(ptr));
    return 0;
}

int trocm_h2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return 0;
    TROCM_NOT_NULL(dst);
    TROCM_NOT_NULL(src);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    TROCM_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s));
    return 0;
}

int trocm_d2h(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return 0;
    TROCM_NOT_NULL(dst);
    TROCM_NOT_NULL(src);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    TROCM_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, s));
    return 0;
}

int trocm_memset(void *dst, int value, size_t bytes, void *stream) {
    if (bytes == 0) return 0;
    TROCM_NOT_NULL(dst);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    TROCM_HIP(hipMemsetAsync(dst, value, bytes, s));
    return 0;
}

int trocm_stream_create(void **stream) {
    TROCM_NOT_NULL(stream);
    if (ensure_init()) return 1;
    hipStream_t s;
    TROCM_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = (void *)s;
    return 0;
}

int trocm_stream_destroy(void *stream) {
    if (!stream) return 0;
    TROCM_HIP(hipStreamDestroy((hipStream_t)stream));
    return 0;
}

int trocm_stream_sync(void *stream) {
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    TROCM_HIP(hipStreamSynchronize(s));
    reap_deferred(false);   // planes that growing caches left behind and nothing reads any more
    return 0;
}

int trocm_device_sync(void) {
    if (ensure_init()) return 1;
    TROCM_HIP(hipDeviceSynchronize());
    reap_deferred(false);
    return 0;
}

int trocm_event_create(void **event) {
    TROCM_NOT_NULL(event);
    if (ensure_init()) return 1;
    hipEvent_t e;
    TROCM_HIP(hipEventCreate(&e));
    *event = (void *)e;
    return 0;
}

int trocm_event_destroy(void *event) {
    if (!event) return 0;
    TROCM_HIP(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int trocm_event_record(void *event, void *stream) {
    TROCM_NOT_NULL(event);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    TROCM_HIP(hipEventRecord((hipEvent_t)event, s));
    return 0;
}

int trocm_event_elapsed_ms(void *start, void *stop, float *ms) {
    TROCM_NOT_NULL(start);
    TROCM_NOT_NULL(stop);
    TROCM_NOT_NULL(ms);
    TROCM_HIP(hipEventSynchronize((hipEvent_t)stop));
    TROCM_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

int trocm_copy_nd(void *dst, size_t dst_offset_bytes, const int64_t *dst_strides, const void *src,
                  size_t src_offset_bytes, const int64_t *src_strides, const int64_t *shape, int rank, int elem_size,
                  void *stream) {
    TROCM_NOT_NULL(dst);
    TROCM_NOT_NULL(src);
    TROCM_NOT_NULL(dst_strides);
    TROCM_NOT_NULL(src_strides);
    TROCM_NOT_NULL(shape);
    TROCM_REQUIRE(rank >= 1 && rank <= 6, "copy_nd: rank %d not in 1..6", rank);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    CopyNd d;
    d.rank = rank;
    for (int i = 0; i < rank; i++) {
        d.shape[i] = shape[i];
        d.dst_stride[i] = dst_strides[i] * elem_size;
        d.src_stride[i] = src_strides[i] * elem_size;
    }
    return launch_copy_nd((char *)dst + dst_offset_bytes, (const char *)src + src_offset_bytes, d, elem_size, s);
}

// ---- KV cache ----------------------------------------------------------------------------------
int trocm_kv_cache_create(trocm_kv_cache **out, int fmt, int64_t batch, int64_t kv_heads, int64_t head_dim) {
    TROCM_NOT_NULL(out);
    if (ensure_init()) return 1;
    TROCM_REQUIRE(fmt >= TROCM_F32 && fmt <= TROCM_Q4_0, "unknown storage format %d", fmt);
    TROCM_REQUIRE(batch >= 1 && kv_heads >= 1 && head_dim >= 1, "kv cache: batch, kv_heads and head_dim must be >= 1");
    TROCM_REQUIRE(!is_quant(fmt) || head_dim % 32 == 0,
                  "quantised KV cache needs head_dim %% 32 == 0, got %lld", (long long)head_dim);
    trocm_kv_cache *c = new (std::nothrow) trocm_kv_cache();
    TROCM_REQUIRE(c != nullptr, "out of host memory");
    c->fmt = fmt;
    c->B = batch, c->H = kv_heads, c->D = head_dim;
    c->len = c->cap = c->reallocs = c->pitch = 0;
    c->data = c->scales = nullptr;
    c->pool = nullptr;
    c->window = c->cursor = 0;
    *out = c;
    return 0;
}

int trocm_kv_cache_create_window(trocm_kv_cache **out, int fmt, int64_t batch, int64_t kv_heads, int64_t head_dim,
                                 int64_t window) {
    TROCM_REQUIRE(window > 0, "window must be > 0");  // window_kv_cache.rs:91
    if (trocm_kv_cache_create(out, fmt, batch, kv_heads, head_dim)) return 1;
    (*out)->window = window;
    return 0;
}

int trocm_kv_cache_window(const trocm_kv_cache *c, int64_t *window, int64_t *cursor) {
    TROCM_NOT_NULL(c);
    if (window) *window = c->window;
    if (cursor) *cursor = c->cursor;
    return 0;
}

int trocm_kv_cache_create_in_pool(trocm_kv_cache **out, trocm_kv_pool *pool, int fmt, int64_t batch, int64_t kv_heads,
                                  int64_t head_dim) {
    TROCM_NOT_NULL(pool);
    if (trocm_kv_cache_create(out, fmt, batch, kv_heads, head_dim)) return 1;
    (*out)->pool = pool;
    std::lock_guard<std::mutex> lock(pool->mu);
    pool->live_caches += 1;
    return 0;
}

int trocm_kv_cache_destroy(trocm_kv_cache *c) {
    if (!c) return 0;
    reap_deferred(false);
    // No stream is known here and kernels queued anywhere may still read the planes: hipFree waits for the device
    // by itself, the pool's bookkeeping does not, so a pooled cache waits explicitly before its planes can be
    // handed to another cache.
    if (c->pool && (c->data || c->scales)) (void)hipDeviceSynchronize();
    int rc = plane_free(c, c->data);
    rc |= plane_free(c, c->scales);
    if (c->pool) {
        std::lock_guard<std::mutex> lock(c->pool->mu);
        c->pool->live_caches -= 1;
    }
    delete c;
    return rc;
}

int trocm_kv_pool_create(trocm_kv_pool **out, size_t bytes) {
    TROCM_NOT_NULL(out);
    if (ensure_init()) return 1;
    TROCM_REQUIRE(bytes >= 256, "kv pool: size must be at least 256 bytes");
    bytes &= ~(size_t)255;
    trocm_kv_pool *p = new (std::nothrow) trocm_kv_pool();
    TROCM_REQUIRE(p != nullptr, "out of host memory");
    hipError_t e = hipMalloc((void **)&p->base, bytes);
    if (e != hipSuccess) {
        delete p;
        return fail("allocating a KV pool of %zu bytes failed: %s", bytes, hipGetErrorString(e));
    }
    p->bytes = bytes;
    p->free_list[0] = bytes;
    *out = p;
    return 0;
}

int trocm_kv_pool_destroy(trocm_kv_pool *p) {
    if (!p) return 0;
    reap_deferred(true, p);
    TROCM_REQUIRE(p->live_caches == 0, "kv pool still has %lld live caches", (long long)p->live_caches);
    TROCM_HIP(hipFree(p->base));
    delete p;
    return 0;
}

int trocm_kv_pool_stats(trocm_kv_pool *p, size_t *bytes_total, size_t *bytes_in_use, size_t *largest_free,
                        void **base) {
    TROCM_NOT_NULL(p);
    reap_deferred(true, p);   // planes left behind by growth count as free once their last reader has finished
    std::lock_guard<std::mutex> lock(p->mu);
    if (bytes_total) *bytes_total = p->bytes;
    if (bytes_in_use) *bytes_in_use = p->in_use;
    if (largest_free) {
        size_t m = 0;
        for (auto &kv : p->free_list) m = kv.second > m ? kv.second : m;
        *largest_free = m;
    }
    if (base) *base = p->base;
    return 0;
}

int trocm_kv_cache_len(const trocm_kv_cache *c, int64_t *len) {
    TROCM_NOT_NULL(c);
    TROCM_NOT_NULL(len);
    *len = c->len;
    return 0;
}
int trocm_kv_cache_capacity(const trocm_kv_cache *c, int64_t *capacity) {
    TROCM_NOT_NULL(c);
    TROCM_NOT_NULL(capacity);
    *capacity = c->cap;
    return 0;
}
int trocm_kv_cache_reallocs(const trocm_kv_cache *c, int64_t *reallocs) {
    TROCM_NOT_NULL(c);
    TROCM_NOT_NULL(reallocs);
    *reallocs = c->reallocs;
    return 0;
}

int trocm_kv_cache_reserve(trocm_kv_cache *c, int64_t capacity, void *stream) {
    TROCM_NOT_NULL(c);
    TROCM_REQUIRE(capacity >= 0, "reserve: negative capacity");
    TROCM_REQUIRE(c->window == 0, "reserve: a sliding-window cache has a fixed capacity of %lld", (long long)c->window);
    if (capacity <= c->cap) return 0;
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return regrow(c, capacity, s);
}

// Argument checks and the growth rule of push (inplace_kv_cache.rs:55-80).
static int append_prepare(trocm_kv_cache *c, const void *src, int src_dtype, const int64_t *src_strides, int64_t n_new,
                          hipStream_t s) {
    TROCM_NOT_NULL(src);
    TROCM_NOT_NULL(src_strides);
    TROCM_REQUIRE(src_dtype == TROCM_F32 || src_dtype == TROCM_F16, "append: source dtype must be F32 or F16");
    TROCM_REQUIRE(is_quant(c->fmt) || src_dtype == c->fmt,
                  "append: source dtype %d does not match the cache's storage format %d", src_dtype, c->fmt);
    for (int i = 0; i < 4; i++) TROCM_REQUIRE(src_strides[i] >= 0, "append: negative source strides are not supported");
    if (c->window) {  // window_kv_cache.rs:101-108: the ring buffer is allocated once, at the window
        if (c->cap == 0 && regrow(c, c->window, s)) return 1;
        return 0;
    }
    if (c->cap == 0) {
        if (regrow(c, n_new, s)) return 1;
    } else if (c->len + n_new > c->cap) {
        int64_t new_cap = c->cap * 2 > c->len + n_new ? c->cap * 2 : c->len + n_new;
        if (regrow(c, new_cap, s)) return 1;
        c->reallocs += 1;
    }
    return 0;
}

// Write source tokens [s0, s0 + n_new) at cache positions [t0, t0 + n_new) (inside the capacity).
static int append_write_at(trocm_kv_cache *c, const void *src0, int src_dtype, const int64_t *src_strides, int64_t s0,
                           int64_t n_new, int64_t t0, hipStream_t s) {
    const void *src = (const char *)src0 + s0 * src_strides[2] * (int64_t)elem_bytes(src_dtype);
    if (is_quant(c->fmt)) {
        QuantAppend a;
        a.fmt = c->fmt, a.src_dtype = src_dtype;
        a.B = c->B, a.H = c->H, a.S = n_new, a.D = c->D;
        for (int i = 0; i < 4; i++) a.ss[i] = src_strides[i];
        a.cap = c->pitch, a.t0 = t0;
        a.src = src, a.codes = c->data, a.scales = c->scales;
        return launch_quant_append(a, s);
    }
    int64_t es = (int64_t)elem_bytes(c->fmt);
    CopyNd d;
    d.rank = 4;
    d.shape[0] = c->B, d.shape[1] = c->H, d.shape[2] = n_new, d.shape[3] = c->D;
    for (int i = 0; i < 4; i++) d.src_stride[i] = src_strides[i] * es;
    d.dst_stride[0] = c->H * c->pitch * c->D * es;
    d.dst_stride[1] = c->pitch * c->D * es;
    d.dst_stride[2] = c->D * es;
    d.dst_stride[3] = es;
    return launch_copy_nd((char *)c->data + t0 * c->D * es, src, d, (int)es, s);
}

// Ring-buffer push of a sliding-window cache (window_kv_cache.rs:111-143).
static int window_write(trocm_kv_cache *c, const void *src, int src_dtype, const int64_t *src_strides, int64_t n_new,
                        hipStream_t s) {
    const int64_t w = c->window;
    if (n_new >= w) {  // only the last w tokens survive, laid out [0, w); the cursor resets
        if (append_write_at(c, src, src_dtype, src_strides, n_new - w, w, 0, s)) return 1;
        c->cursor = 0;
        c->len = w;
        return 0;
    }
    const int64_t end = c->cursor + n_new;
    if (end <= w) {
        if (append_write_at(c, src, src_dtype, src_strides, 0, n_new, c->cursor, s)) return 1;
        c->cursor = end == w ? 0 : end;
    } else {
        const int64_t first = w - c->cursor;
        if (append_write_at(c, src, src_dtype, src_strides, 0, first, c->cursor, s)) return 1;
        if (append_write_at(c, src, src_dtype, src_strides, first, n_new - first, 0, s)) return 1;
        c->cursor = n_new - first;
    }
    c->len = c->len + n_new < w ? c->len + n_new : w;
    return 0;
}

// Write the new tokens at [len, len + n_new) (capacity is already sufficient).
static int append_write(trocm_kv_cache *c, const void *src, int src_dtype, const int64_t *src_strides, int64_t n_new,
                        hipStream_t s) {
    return append_write_at(c, src, src_dtype, src_strides, 0, n_new, c->len, s);
}

int trocm_kv_append(trocm_kv_cache *c, const void *src, int src_dtype, const int64_t *src_strides, int64_t n_new,
                    void *stream) {
    TROCM_NOT_NULL(c);
    TROCM_REQUIRE(n_new >= 0, "append: negative token count");
    if (n_new == 0) return 0;  // inplace_kv_cache.rs:57-59
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    if (append_prepare(c, src, src_dtype, src_strides, n_new, s)) return 1;
    if (c->window) return window_write(c, src, src_dtype, src_strides, n_new, s);
    if (append_write(c, src, src_dtype, src_strides, n_new, s)) return 1;
    c->len += n_new;
    return 0;
}

int trocm_kv_append_pair(trocm_kv_cache *kc, trocm_kv_cache *vc, const void *k_src, const void *v_src, int src_dtype,
                         const int64_t *src_strides, int64_t n_new, void *stream) {
    TROCM_NOT_NULL(kc);
    TROCM_NOT_NULL(vc);
    TROCM_REQUIRE(n_new >= 0, "append: negative token count");
    TROCM_REQUIRE(kc->fmt == vc->fmt && kc->B == vc->B && kc->H == vc->H && kc->D == vc->D,
                  "K and V caches differ in format or shape");
    if (n_new == 0) return 0;
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    TROCM_REQUIRE(kc->window == vc->window, "K and V caches differ in window");
    TROCM_NOT_NULL(k_src);
    TROCM_NOT_NULL(v_src);
    if (kc->len == vc->len && equalise_capacities(kc, vc, s)) return 1;
    if (append_prepare(kc, k_src, src_dtype, src_strides, n_new, s)) return 1;
    if (append_prepare(vc, v_src, src_dtype, src_strides, n_new, s)) return 1;
    if (kc->window) {
        if (window_write(kc, k_src, src_dtype, src_strides, n_new, s)) return 1;
        return window_write(vc, v_src, src_dtype, src_strides, n_new, s);
    }
    int rc = 2;
    if (!is_quant(kc->fmt) && src_strides[3] == 1 && kc->cap == vc->cap && kc->len == vc->len) {
        int64_t es = (int64_t)elem_bytes(kc->fmt);
        AppendPair a;
        a.src[0] = k_src, a.src[1] = v_src;
        a.dst[0] = (char *)kc->data + kc->len * kc->D * es;
        a.dst[1] = (char *)vc->data + vc->len * vc->D * es;
        a.B = kc->B, a.H = kc->H, a.S = n_new, a.row_bytes = kc->D * es;
        for (int i = 0; i < 3; i++) a.src_stride[i] = src_strides[i] * es;
        a.dst_stride[0] = kc->H * kc->pitch * kc->D * es, a.dst_stride[1] = kc->pitch * kc->D * es, a.dst_stride[2] = kc->D * es;
        rc = launch_append_pair(a, s);
    }
    if (is_quant(kc->fmt)) {   // both tensors quantised by one launch
        QuantAppend a[2];
        trocm_kv_cache *cs[2] = {kc, vc};
        const void *srcs[2] = {k_src, v_src};
        for (int t = 0; t < 2; t++) {
            a[t].fmt = cs[t]->fmt, a[t].src_dtype = src_dtype;
            a[t].B = cs[t]->B, a[t].H = cs[t]->H, a[t].S = n_new, a[t].D = cs[t]->D;
            for (int i = 0; i < 4; i++) a[t].ss[i] = src_strides[i];
            a[t].cap = cs[t]->pitch, a[t].t0 = cs[t]->len;
            a[t].src = srcs[t], a[t].codes = cs[t]->data, a[t].scales = cs[t]->scales;
        }
        rc = launch_quant_append_pair(a[0], a[1], s);
    }
    if (rc == 2) {
        rc = append_write(kc, k_src, src_dtype, src_strides, n_new, s);
        if (!rc) rc = append_write(vc, v_src, src_dtype, src_strides, n_new, s);
    }
    if (rc) return rc;
    kc->len += n_new;
    vc->len += n_new;
    return 0;
}

int trocm_kv_cache_truncate(trocm_kv_cache *c, int64_t len) {
    TROCM_NOT_NULL(c);
    TROCM_REQUIRE(c->data != nullptr, "Can not truncate a zero-len kv-cache value");  // dyn_kv_cache.rs:112-119
    TROCM_REQUIRE(c->window == 0, "truncate: a sliding-window cache does not keep its tokens in order");
    TROCM_REQUIRE(len >= 0 && len <= c->len, "truncate: length %lld out of range 0..=%lld", (long long)len,
                  (long long)c->len);
    c->len = len;
    return 0;
}

int trocm_kv_row_bytes(const trocm_kv_cache *c, size_t *bytes) {
    TROCM_NOT_NULL(c);
    TROCM_NOT_NULL(bytes);
    *bytes = canonical_row_bytes(c->fmt, c->D);
    return 0;
}

int trocm_kv_export(const trocm_kv_cache *c, void *dst, void *stream) {
    TROCM_NOT_NULL(c);
    if (c->len == 0) return 0;
    TROCM_NOT_NULL(dst);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    if (is_quant(c->fmt))
        return launch_quant_export(c->fmt, c->B, c->H, c->len, c->pitch, c->D, c->data, c->scales, dst, s);
    CopyNd d;
    d.rank = 2;
    int64_t rb = (int64_t)device_row_bytes(c->fmt, c->D);
    d.shape[0] = c->B * c->H;
    d.shape[1] = c->len * rb;
    d.dst_stride[0] = c->len * rb;
    d.src_stride[0] = c->pitch * rb;
    d.dst_stride[1] = d.src_stride[1] = 1;
    return launch_copy_nd(dst, c->data, d, 1, s);
}

int trocm_kv_cache_clone(const trocm_kv_cache *c, trocm_kv_cache **out, void *stream) {
    TROCM_NOT_NULL(c);
    TROCM_NOT_NULL(out);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    trocm_kv_cache *n = nullptr;
    if (c->pool ? trocm_kv_cache_create_in_pool(&n, c->pool, c->fmt, c->B, c->H, c->D)
                : trocm_kv_cache_create(&n, c->fmt, c->B, c->H, c->D))
        return 1;
    if (c->cap) {
        if (regrow(n, c->cap, s)) {
            trocm_kv_cache_destroy(n);
            return 1;
        }
        if (copy_valid(c, n->data, n->scales, n->pitch, c->data, c->scales, c->pitch, c->len, s)) {
            trocm_kv_cache_destroy(n);
            return 1;
        }
    }
    n->len = c->len;
    n->reallocs = c->reallocs;
    n->window = c->window, n->cursor = c->cursor;
    *out = n;
    return 0;
}

// Append `n_tokens` tokens given as canonical blocks on the device ([batch, kv_heads, n_tokens,
// head_dim/32 * block_bytes], what trocm_kv_export writes): load_from of a quantised state without
// a round trip through floats.
int trocm_kv_import_blocks(trocm_kv_cache *c, const void *blocks, int64_t n_tokens, void *stream) {
    TROCM_NOT_NULL(c);
    TROCM_REQUIRE(is_quant(c->fmt), "import_blocks: the cache stores plain %s tensors, append them instead",
                  c->fmt == TROCM_F32 ? "f32" : "f16");
    TROCM_REQUIRE(c->window == 0, "import_blocks: not supported for a sliding-window cache");
    TROCM_REQUIRE(n_tokens >= 0, "import_blocks: negative token count");
    if (n_tokens == 0) return 0;
    TROCM_NOT_NULL(blocks);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    if (c->cap == 0) {
        if (regrow(c, n_tokens, s)) return 1;
    } else if (c->len + n_tokens > c->cap) {
        int64_t new_cap = c->cap * 2 > c->len + n_tokens ? c->cap * 2 : c->len + n_tokens;
        if (regrow(c, new_cap, s)) return 1;
        c->reallocs += 1;
    }
    if (launch_quant_import(c->fmt, c->B, c->H, n_tokens, c->pitch, c->len, c->D, blocks, c->data, c->scales, s)) return 1;
    c->len += n_tokens;
    return 0;
}

int trocm_kv_cache_raw(const trocm_kv_cache *c, void **data, void **scales, int64_t *capacity) {
    TROCM_NOT_NULL(c);
    if (data) *data = c->data;
    if (scales) *scales = c->scales;
    if (capacity) *capacity = c->pitch;
    return 0;
}

// ---- Q4_0 weights and the decode-time projection --------------------------------------------------
}  // extern "C" (the struct below is opaque to C callers)

struct trocm_q4_weights {
    int64_t batch, n, k;
    void *codes, *scales;   // [batch * n, k/2] bytes and [batch * n, k/32] f16
    int tiled;              // codes = tiles of 16 rows x 128 features with their scales (q4_tiled.hip), scales = NULL
    // A small tiled matrix (up to 3072 rows: the key / value projections of a decoder with grouped heads) keeps the
    // planes as well: its 16-row tiles give the matrix-instruction kernel too few independent pieces for the compute
    // units, and one or two activation rows run faster over the planes, a wave per row (1024 x 4096: 3.7 against 4.8 us).
    void *row_codes, *row_scales;
};

extern "C" {

int trocm_q4_0_weights_create(trocm_q4_weights **out, const void *blocks, int64_t batch, int64_t n, int64_t k,
                              void *stream) {
    TROCM_NOT_NULL(out);
    *out = nullptr;
    TROCM_REQUIRE(batch >= 1 && n >= 1 && k >= 32, "q4_0 weights: empty shape [%lld, %lld, %lld]", (long long)batch,
                  (long long)n, (long long)k);
    TROCM_REQUIRE(k % 32 == 0, "q4_0 weights: k = %lld is not a whole number of 32-element blocks", (long long)k);  // utils.rs:253
    TROCM_REQUIRE(batch * n < (1ll << 31) && k < (1ll << 31), "q4_0 weights: shape too large");
    TROCM_NOT_NULL(blocks);
    if (ensure_init()) return 1;
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    trocm_q4_weights *w = new (std::nothrow) trocm_q4_weights();
    TROCM_REQUIRE(w != nullptr, "out of host memory");
    w->batch = batch, w->n = n, w->k = k;
    const int64_t rows = batch * n;
    // The matrices of a decoder (rows a multiple of 16, features of 128) are tiled for the matrix instruction;
    // TROCM_Q4_TILED=0 (read at every call) keeps the planes of codes and scales for them too.
    const char *tiled_env = getenv("TROCM_Q4_TILED");
    w->tiled = q4_0_tiled_layout_fits(n, k) && !(tiled_env && atoi(tiled_env) == 0);
    hipError_t e = hipMalloc(&w->codes, w->tiled ? q4_0_tiled_bytes(rows, k) : (size_t)rows * (size_t)(k / 2));
    if (e == hipSuccess && !w->tiled) e = hipMalloc(&w->scales, (size_t)rows * (size_t)(k / 32) * 2);
    if (e != hipSuccess) {
        if (w->codes) (void)hipFree(w->codes);
        delete w;
        return fail("q4_0 weights: hipMalloc failed: %s", hipGetErrorString(e));
    }
    // TROCM_Q4_ROWS_TOO=0 (read at every call): tiles only, whatever the size
    const char *rows_env = getenv("TROCM_Q4_ROWS_TOO");
    const bool rows_too = w->tiled && n <= 3072 && !(rows_env && atoi(rows_env) == 0);
    if (e == hipSuccess && rows_too) {
        e = hipMalloc(&w->row_codes, (size_t)rows * (size_t)(k / 2));
        if (e == hipSuccess) e = hipMalloc(&w->row_scales, (size_t)rows * (size_t)(k / 32) * 2);
        if (e != hipSuccess) {
            (void)hipFree(w->codes);
            if (w->row_codes) (void)hipFree(w->row_codes);
            delete w;
            return fail("q4_0 weights: hipMalloc failed: %s", hipGetErrorString(e));
        }
    }
    if ((w->tiled ? launch_q4_0_tiled_import(blocks, w->codes, rows, k, s)
                  : launch_quant_import(TROCM_Q4_0, 1, 1, rows, rows, 0, k, blocks, w->codes, w->scales, s)) ||
        (rows_too && launch_quant_import(TROCM_Q4_0, 1, 1, rows, rows, 0, k, blocks, w->row_codes, w->row_scales, s))) {
        (void)hipFree(w->codes);
        if (w->scales) (void)hipFree(w->scales);
        if (w->row_codes) (void)hipFree(w->row_codes);
        if (w->row_scales) (void)hipFree(w->row_scales);
        delete w;
        return 1;
    }
    *out = w;
    return 0;
}

int trocm_q4_0_weights_destroy(trocm_q4_weights *w) {
    if (!w) return 0;
    TROCM_HIP(hipDeviceSynchronize());
    TROCM_HIP(hipFree(w->codes));
    if (w->scales) TROCM_HIP(hipFree(w->scales));
    if (w->row_codes) TROCM_HIP(hipFree(w->row_codes));
    if (w->row_scales) TROCM_HIP(hipFree(w->row_scales));
    delete w;
    return 0;
}

int trocm_q4_0_weights_shape(const trocm_q4_weights *w, int64_t *batch, int64_t *n, int64_t *k) {
    TROCM_NOT_NULL(w);
    if (batch) *batch = w->batch;
    if (n) *n = w->n;
    if (k) *k = w->k;
    return 0;
}

int trocm_q4_0_weights_export(const trocm_q4_weights *w, void *dst_blocks, void *stream) {
    TROCM_NOT_NULL(w);
    TROCM_NOT_NULL(dst_blocks);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    const int64_t rows = w->batch * w->n;
    if (w->tiled) return launch_q4_0_tiled_export(w->codes, dst_blocks, rows, w->k, s);
    return launch_quant_export(TROCM_Q4_0, 1, 1, rows, rows, w->k, w->codes, w->scales, dst_blocks, s);
}

int trocm_q4_0_matvec(const trocm_q4_weights *w, const void *act, int act_dtype, int64_t act_batch, int64_t m, void *out,
                      void *stream) {
    TROCM_NOT_NULL(w);
    TROCM_REQUIRE(act_dtype == TROCM_F32 || act_dtype == TROCM_F16, "q4_0_matvec: activations must be F32 or F16");
    TROCM_REQUIRE(act_batch >= 0 && m >= 0, "q4_0_matvec: negative dimension");
    if (act_batch == 0 || m == 0) return 0;                                      // mod.rs:586-588
    TROCM_REQUIRE(act_batch % w->batch == 0, "q4_0_matvec: activation batch %lld is not a multiple of the weights' batch %lld",
                  (long long)act_batch, (long long)w->batch);                     // mod.rs:488
    TROCM_REQUIRE(act_batch <= 65535, "q4_0_matvec: batch too large");
    TROCM_NOT_NULL(act);
    TROCM_NOT_NULL(out);
    TROCM_REQUIRE((uintptr_t)act % 16 == 0, "q4_0_matvec: activations must be 16-byte aligned");
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    if (w->tiled && w->row_codes && m <= 2)
        return launch_q4_0_matvec(w->row_codes, w->row_scales, w->batch, w->n, w->k, act, act_dtype, act_batch, m, out, s);
    if (w->tiled) return launch_q4_0_tiled_matvec(w->codes, w->batch, w->n, w->k, act, act_dtype, act_batch, m, out, s);
    return launch_q4_0_matvec(w->codes, w->scales, w->batch, w->n, w->k, act, act_dtype, act_batch, m, out, s);
}

// ---- block quantisation as a tensor op ---------------------------------------------------------
int trocm_block_quant(int format, const void *src, int src_dtype, size_t n_elems, void *dst_blocks, void *stream) {
    TROCM_REQUIRE(format == TROCM_Q8_0 || format == TROCM_Q4_0, "block_quant: format must be Q8_0 or Q4_0");
    TROCM_REQUIRE(src_dtype == TROCM_F32 || src_dtype == TROCM_F16, "block_quant: source dtype must be F32 or F16");
    TROCM_REQUIRE(n_elems % 32 == 0, "block_quant: %zu elements is not a multiple of the block length 32", n_elems);
    if (n_elems == 0) return 0;
    TROCM_NOT_NULL(src);
    TROCM_NOT_NULL(dst_blocks);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return launch_block_quant(format, src, src_dtype, n_elems, dst_blocks, s);
}

int trocm_block_dequant(int format, const void *src_blocks, size_t n_elems, void *dst, int dst_dtype, void *stream) {
    TROCM_REQUIRE(format == TROCM_Q8_0 || format == TROCM_Q4_0, "block_dequant: format must be Q8_0 or Q4_0");
    TROCM_REQUIRE(dst_dtype == TROCM_F32 || dst_dtype == TROCM_F16, "block_dequant: output dtype must be F32 or F16");
    TROCM_REQUIRE(n_elems % 32 == 0, "block_dequant: %zu elements is not a multiple of the block length 32", n_elems);
    if (n_elems == 0) return 0;
    TROCM_NOT_NULL(src_blocks);
    TROCM_NOT_NULL(dst);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return launch_block_dequant(format, src_blocks, n_elems, dst, dst_dtype, s);
}

int trocm_block_simulate_precision_loss(int format, const void *src, void *dst, int dtype, size_t n_elems, void *stream) {
    TROCM_REQUIRE(format == TROCM_Q8_0 || format == TROCM_Q4_0, "simulate_precision_loss: format must be Q8_0 or Q4_0");
    TROCM_REQUIRE(dtype == TROCM_F32 || dtype == TROCM_F16, "simulate_precision_loss: dtype must be F32 or F16");
    TROCM_REQUIRE(n_elems % 32 == 0, "simulate_precision_loss: %zu elements is not a multiple of the block length 32", n_elems);
    if (n_elems == 0) return 0;
    TROCM_NOT_NULL(src);
    TROCM_NOT_NULL(dst);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return launch_block_simulate(format, src, dst, dtype, n_elems, s);
}

int trocm_release_unused(int wait) {
    if (ensure_init()) return 1;
    reap_deferred(wait != 0);
    return 0;
}

// ---- launch floors -----------------------------------------------------------------------------
int trocm_launch_floor(int kind, const void *src, size_t bytes, int workgroups, int threads, void *sink, void *stream) {
    if (ensure_init()) return 1;
    TROCM_REQUIRE(kind == 0 || kind == 1, "launch_floor: kind is 0 (empty kernel) or 1 (streaming read), got %d", kind);
    TROCM_REQUIRE(workgroups >= 1 && workgroups <= (1 << 20) && threads >= 64 && threads <= 1024 && threads % 64 == 0,
                  "launch_floor: %d workgroups of %d threads is not a launch shape (1..2^20 workgroups of 64..1024 threads in whole waves)",
                  workgroups, threads);
    if (kind == 1) {
        TROCM_NOT_NULL(src);
        TROCM_REQUIRE((uintptr_t)src % 16 == 0 && bytes % 16 == 0, "launch_floor: the buffer must be 16-byte aligned and a multiple of 16 bytes");
    }
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return launch_floor(kind, src, bytes, workgroups, threads, sink, s);
}

// ---- element-wise neighbours: cast, RotateHalf, ApplyRope ---------------------------------------
int trocm_cast(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n_elems, void *stream) {
    TROCM_REQUIRE((src_dtype == TROCM_F32 || src_dtype == TROCM_F16) && (dst_dtype == TROCM_F32 || dst_dtype == TROCM_F16),
                  "cast: only F32 and F16 are handled here (got %d -> %d)", src_dtype, dst_dtype);
    if (n_elems == 0) return 0;
    TROCM_NOT_NULL(src);
    TROCM_NOT_NULL(dst);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return launch_cast(src, src_dtype, dst, dst_dtype, n_elems, s);
}

static int rope_common(const void *input, const void *cos, const void *sin, void *out, int dtype, int rank,
                       const int64_t *shape, const int64_t *in_strides, const int64_t *cs_strides,
                       const int64_t *out_strides, int rotate_only, void *stream) {
    const char *what = rotate_only ? "rotate_half" : "apply_rope";
    TROCM_REQUIRE(dtype == TROCM_F32 || dtype == TROCM_F16, "Unsupported dt %d for %s", dtype, what);
    TROCM_NOT_NULL(shape);
    // apply_rope.rs (cuda kernels) :72-73: rank 2..4; RotateHalf takes any rank >= 1 (here up to 4)
    TROCM_REQUIRE(rank >= (rotate_only ? 1 : 2) && rank <= 4, "%s: unsupported rank %d", what, rank);
    int64_t n = 1;
    for (int d = 0; d < rank; d++) {
        TROCM_REQUIRE(shape[d] >= 0, "%s: negative dimension", what);
        n *= shape[d];
    }
    TROCM_REQUIRE(shape[rank - 1] % 2 == 0,
                  "RotateHalf possible only if the most inner dimension of the shape is divisible by 2 (got %lld)",
                  (long long)shape[rank - 1]);  // apply_rope.rs:64-68
    if (n == 0) return 0;
    TROCM_NOT_NULL(input);
    TROCM_NOT_NULL(out);
    if (!rotate_only) {
        TROCM_NOT_NULL(cos);
        TROCM_NOT_NULL(sin);
    }
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return launch_apply_rope(input, cos, sin, out, dtype, rank, shape, in_strides, cs_strides, out_strides, rotate_only, s);
}

int trocm_apply_rope(const void *input, const void *cos, const void *sin, void *out, int dtype, int rank,
                     const int64_t *shape, const int64_t *in_strides, const int64_t *cos_sin_strides,
                     const int64_t *out_strides, void *stream) {
    return rope_common(input, cos, sin, out, dtype, rank, shape, in_strides, cos_sin_strides, out_strides, 0, stream);
}

int trocm_rotate_half(const void *input, void *out, int dtype, int rank, const int64_t *shape,
                      const int64_t *in_strides, const int64_t *out_strides, void *stream) {
    return rope_common(input, nullptr, nullptr, out, dtype, rank, shape, in_strides, nullptr, out_strides, 1, stream);
}

// ---- attention -----------------------------------------------------------------------------------
int trocm_sdpa_workspace_bytes(int64_t batch, int64_t q_heads, int64_t q_len, int64_t head_dim, size_t *bytes) {
    TROCM_NOT_NULL(bytes);
    TROCM_REQUIRE(batch >= 0 && q_heads >= 0 && q_len >= 0 && head_dim >= 0, "workspace_bytes: negative dimension");
    size_t need = decode_workspace_bytes(batch, q_heads, head_dim);
    size_t prefill = kWsCounterBytes + prefill_workspace_bytes(batch, q_heads, q_len, head_dim);
    *bytes = need > prefill ? need : prefill;
    return 0;
}

int trocm_sdpa_workspace_init(void *workspace, size_t bytes, void *stream) {
    TROCM_NOT_NULL(workspace);
    TROCM_REQUIRE(bytes >= kWsCounterBytes, "workspace of %zu bytes is smaller than the counter area", bytes);
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    TROCM_HIP(hipMemsetAsync(workspace, 0, kWsCounterBytes, s));
    return 0;
}

static int dispatch_sdpa(const SdpaArgs &a, hipStream_t s) {
    if (a.B == 0 || a.Hq == 0 || a.Sq == 0 || a.D == 0) return 0;
    int rc = 2;
    if (a.Sq == 1) rc = is_quant(a.kv_fmt) ? launch_sdpa_decode_quant(a, s) : launch_sdpa_decode(a, s);
    if (rc == 2 && a.Sq > 1) rc = launch_sdpa_prefill_pp(a, s);
    if (rc == 2) rc = launch_sdpa_prefill(a, s);
    if (rc == 2) rc = launch_sdpa_generic(a, s);
    return rc;
}

int trocm_sdpa(const void *q, const void *k, const void *v, const void *mask, void *out, int dtype, int64_t batch,
               int64_t q_heads, int64_t kv_heads, int64_t q_len, int64_t kv_len, int64_t head_dim,
               const int64_t *kv_strides, int64_t mask_batch, int64_t mask_heads, float scale, int causal,
               void *workspace, size_t workspace_bytes, void *stream) {
    TROCM_NOT_NULL(q);
    TROCM_NOT_NULL(k);
    TROCM_NOT_NULL(v);
    TROCM_NOT_NULL(out);
    TROCM_REQUIRE(dtype == TROCM_F32 || dtype == TROCM_F16, "sdpa: dtype must be F32 or F16");
    TROCM_REQUIRE(batch >= 0 && q_heads >= 0 && kv_heads >= 1 && q_len >= 0 && kv_len >= 0 && head_dim >= 0,
                  "sdpa: negative dimension");
    TROCM_REQUIRE(q_heads % kv_heads == 0, "Q heads (%lld) must be a multiple of K/V heads (%lld)", (long long)q_heads,
                  (long long)kv_heads);  // sdpa.rs:325-330
    TROCM_REQUIRE(!(causal && mask), "Mask cannot be provided if is_causal=true");  // sdpa.rs:297-299
    if (mask) {
        TROCM_REQUIRE(mask_batch == 1 || mask_batch == batch, "sdpa: mask batch must be 1 or %lld", (long long)batch);
        TROCM_REQUIRE(mask_heads == 1 || mask_heads == q_heads, "sdpa: mask heads must be 1 or %lld", (long long)q_heads);
    }
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    SdpaArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q, a.out = out, a.q_dtype = dtype, a.kv_fmt = dtype;
    a.k = k, a.v = v;
    a.B = batch, a.Hq = q_heads, a.Hkv = kv_heads, a.Sq = q_len, a.Sk = kv_len, a.D = head_dim;
    if (kv_strides) {
        a.kv_stride_b = kv_strides[0], a.kv_stride_h = kv_strides[1], a.kv_stride_t = kv_strides[2];
        TROCM_REQUIRE(a.kv_stride_b >= 0 && a.kv_stride_h >= 0 && a.kv_stride_t >= 0, "sdpa: negative K/V strides");
    } else {
        a.kv_stride_t = head_dim, a.kv_stride_h = kv_len * head_dim, a.kv_stride_b = kv_heads * kv_len * head_dim;
    }
    a.mask = mask, a.mask_b = mask ? mask_batch : 1, a.mask_h = mask ? mask_heads : 1;
    a.scale = isnan(scale) ? 1.0f / sqrtf((float)head_dim) : scale;  // sdpa.rs:177-181
    a.causal = causal;
    a.workspace = workspace, a.workspace_bytes = workspace_bytes;
    if (kv_len == 0) {  // nothing to attend to: zeros, like the CPU op's zero-initialised output (flash_sdpa.rs:253)
        TROCM_HIP(hipMemsetAsync(out, 0, (size_t)batch * q_heads * q_len * head_dim * elem_bytes(dtype), s));
        return 0;
    }
    return dispatch_sdpa(a, s);
}

// Argument checks of an attention call over two caches (none of them touches the device).
static int sdpa_cached_check(const void *q, int q_dtype, int64_t q_heads, const trocm_kv_cache *kc, const trocm_kv_cache *vc,
                             const void *out) {
    TROCM_NOT_NULL(q);
    TROCM_NOT_NULL(kc);
    TROCM_NOT_NULL(vc);
    TROCM_NOT_NULL(out);
    TROCM_REQUIRE(q_dtype == TROCM_F32 || q_dtype == TROCM_F16, "sdpa: q dtype must be F32 or F16");
    TROCM_REQUIRE(kc->fmt == vc->fmt && kc->B == vc->B && kc->H == vc->H && kc->D == vc->D,
                  "K and V caches differ in format or shape");
    TROCM_REQUIRE(kc->len == vc->len, "K/V lengths must match (%lld vs %lld)", (long long)kc->len, (long long)vc->len);
    TROCM_REQUIRE(kc->cap == vc->cap, "K/V capacities must match (%lld vs %lld)", (long long)kc->cap, (long long)vc->cap);
    TROCM_REQUIRE(kc->len > 0, "empty kv-cache");  // inplace_kv_cache.rs:91
    TROCM_REQUIRE(q_heads >= 1 && q_heads % kc->H == 0, "Q heads (%lld) must be a multiple of K/V heads (%lld)", (long long)q_heads,
                  (long long)kc->H);
    TROCM_REQUIRE(is_quant(kc->fmt) || kc->fmt == q_dtype, "q dtype %d does not match the cache format %d", q_dtype,
                  kc->fmt);
    return 0;
}

static int sdpa_cached_run(const void *q, int q_dtype, int64_t q_heads, int64_t q_len, const trocm_kv_cache *kc,
                           const trocm_kv_cache *vc, void *out, float scale, int causal, void *workspace,
                           size_t workspace_bytes, hipStream_t s) {
    SdpaArgs a;
    memset(&a, 0, sizeof(a));
    a.q = q, a.out = out, a.q_dtype = q_dtype, a.kv_fmt = kc->fmt;
    a.k = kc->data, a.v = vc->data, a.k_scales = kc->scales, a.v_scales = vc->scales;
    a.B = kc->B, a.Hq = q_heads, a.Hkv = kc->H, a.Sq = q_len, a.Sk = kc->len, a.D = kc->D;
    a.kv_stride_t = kc->D, a.kv_stride_h = kc->pitch * kc->D, a.kv_stride_b = kc->H * kc->pitch * kc->D;
    a.mask_b = a.mask_h = 1;
    a.scale = isnan(scale) ? 1.0f / sqrtf((float)kc->D) : scale;
    a.causal = causal;
    a.workspace = workspace, a.workspace_bytes = workspace_bytes;
    return dispatch_sdpa(a, s);
}

int trocm_sdpa_cached(const void *q, int q_dtype, int64_t q_heads, int64_t q_len, const trocm_kv_cache *kc,
                      const trocm_kv_cache *vc, void *out, float scale, int causal, void *workspace,
                      size_t workspace_bytes, void *stream) {
    if (sdpa_cached_check(q, q_dtype, q_heads, kc, vc, out)) return 1;
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    return sdpa_cached_run(q, q_dtype, q_heads, q_len, kc, vc, out, scale, causal, workspace, workspace_bytes, s);
}

// trocm_sdpa_cached for callers that cannot allocate: the split-K scratch is the library's static device
// array instead of a caller's workspace, and nothing on this path calls an allocating routine (the caller's
// stream is required because the library's own per-thread stream is created on first use).
int trocm_sdpa_cached_noalloc(const void *q, int q_dtype, int64_t q_heads, int64_t q_len, const trocm_kv_cache *kc,
                              const trocm_kv_cache *vc, void *out, float scale, int causal, void *stream) {
    if (ensure_init()) return 1;
    TROCM_REQUIRE(stream != nullptr, "sdpa_cached_noalloc: a stream is required (the library's per-thread stream would be created here)");
    if (sdpa_cached_check(q, q_dtype, q_heads, kc, vc, out)) return 1;
    TROCM_REQUIRE(q_len >= 0, "sdpa: negative dimension");
    size_t need = 0;
    if (trocm_sdpa_workspace_bytes(kc->B, q_heads, q_len, kc->D, &need)) return 1;
    TROCM_REQUIRE(need <= (size_t)TROCM_STATIC_SCRATCH_BYTES,
                  "sdpa_cached_noalloc: batch %lld x %lld query heads x %lld queries at head_dim %lld asks for %zu bytes of split-K "
                  "scratch, the static buffer holds %zu; call trocm_sdpa_cached with a workspace of that size instead",
                  (long long)kc->B, (long long)q_heads, (long long)q_len, (long long)kc->D, need, (size_t)TROCM_STATIC_SCRATCH_BYTES);
    return sdpa_cached_run(q, q_dtype, q_heads, q_len, kc, vc, out, scale, causal, g_scratch_ptr, (size_t)TROCM_STATIC_SCRATCH_BYTES,
                           (hipStream_t)stream);
}

// Shared argument block of an attention call over two caches.
static void cached_args(SdpaArgs &a, const void *q, int q_dtype, int64_t q_heads, int64_t q_len,
                        const trocm_kv_cache *kc, const trocm_kv_cache *vc, int64_t kv_len, void *out, float scale,
                        int causal, void *workspace, size_t workspace_bytes) {
    memset(&a, 0, sizeof(a));
    a.q = q, a.out = out, a.q_dtype = q_dtype, a.kv_fmt = kc->fmt;
    a.k = kc->data, a.v = vc->data, a.k_scales = kc->scales, a.v_scales = vc->scales;
    a.B = kc->B, a.Hq = q_heads, a.Hkv = kc->H, a.Sq = q_len, a.Sk = kv_len, a.D = kc->D;
    a.kv_stride_t = kc->D, a.kv_stride_h = kc->pitch * kc->D, a.kv_stride_b = kc->H * kc->pitch * kc->D;
    a.mask_b = a.mask_h = 1;
    a.scale = isnan(scale) ? 1.0f / sqrtf((float)kc->D) : scale;
    a.causal = causal;
    a.workspace = workspace, a.workspace_bytes = workspace_bytes;
}

// Everything an append + attention call can be refused for, checked before either cache is touched: a call that
// fails leaves the caches as they were and can be repeated.
static int inplace_eval_check(const char *what, const void *q, const void *k_new, const void *v_new, const void *out, int dtype,
                              int64_t q_heads, int64_t n_new, const trocm_kv_cache *kc, const trocm_kv_cache *vc) {
    TROCM_NOT_NULL(kc);
    TROCM_NOT_NULL(vc);
    TROCM_NOT_NULL(q);
    TROCM_NOT_NULL(k_new);
    TROCM_NOT_NULL(v_new);
    TROCM_NOT_NULL(out);
    TROCM_REQUIRE(dtype == TROCM_F32 || dtype == TROCM_F16, "%s: dtype must be F32 or F16", what);
    TROCM_REQUIRE(n_new >= 0, "append: negative token count");
    TROCM_REQUIRE(kc->fmt == vc->fmt && kc->B == vc->B && kc->H == vc->H && kc->D == vc->D,
                  "K and V caches differ in format or shape");
    TROCM_REQUIRE(kc->window == vc->window, "K and V caches differ in window");
    TROCM_REQUIRE(kc->len == vc->len, "K/V lengths must match (%lld vs %lld)", (long long)kc->len, (long long)vc->len);
    TROCM_REQUIRE(is_quant(kc->fmt) || kc->fmt == dtype, "q dtype %d does not match the cache format %d", dtype, kc->fmt);
    TROCM_REQUIRE(q_heads >= 1 && q_heads % kc->H == 0, "Q heads (%lld) must be a multiple of K/V heads (%lld)", (long long)q_heads,
                  (long long)kc->H);
    TROCM_REQUIRE(kc->len + n_new > 0, "empty kv-cache");  // inplace_kv_cache.rs:91
    return 0;
}

int trocm_inplace_kv_sdpa_eval(const void *q, const void *k_new, const void *v_new, int dtype, int64_t q_heads,
                               int64_t n_new, const int64_t *kv_new_strides, trocm_kv_cache *kc, trocm_kv_cache *vc,
                               void *out, float scale, int causal, void *workspace, size_t workspace_bytes,
                               void *stream) {
    if (inplace_eval_check("inplace_kv_sdpa", q, k_new, v_new, out, dtype, q_heads, n_new, kc, vc)) return 1;
    if (kv_new_strides)
        for (int i = 0; i < 4; i++) TROCM_REQUIRE(kv_new_strides[i] >= 0, "append: negative source strides are not supported");
    {
        hipStream_t s0;
        if (resolve_stream(stream, &s0)) return 1;
        if (equalise_capacities(kc, vc, s0)) return 1;
    }
    int64_t dense[4];
    dense[3] = 1, dense[2] = kc->D, dense[1] = n_new * kc->D, dense[0] = kc->H * n_new * kc->D;
    bool is_dense = kv_new_strides == nullptr;
    if (!is_dense) {
        is_dense = true;
        for (int i = 0; i < 4; i++) is_dense = is_dense && kv_new_strides[i] == dense[i];
    } else {
        kv_new_strides = dense;
    }
    // Decode step: the attention kernel reads the new token from the inputs and stores it into the cache itself (a
    // block-quantised cache: quantises it, f16 inputs) -- one launch instead of append + attention.
    if (n_new == 1 && is_dense && (is_quant(kc->fmt) ? dtype == TROCM_F16 : dtype == kc->fmt) && q && k_new && v_new && out &&
        kc->window == 0 && vc->window == 0 && kc->fmt == vc->fmt && kc->B == vc->B && kc->H == vc->H && kc->D == vc->D && kc->len == vc->len &&
        q_heads % kc->H == 0) {
        hipStream_t s;
        if (resolve_stream(stream, &s)) return 1;
        if (append_prepare(kc, k_new, dtype, kv_new_strides, 1, s)) return 1;
        if (append_prepare(vc, v_new, dtype, kv_new_strides, 1, s)) return 1;
        if (kc->cap == vc->cap) {
            SdpaArgs a;
            cached_args(a, q, dtype, q_heads, 1, kc, vc, kc->len + 1, out, scale, causal, workspace, workspace_bytes);
            a.k_new = k_new, a.v_new = v_new, a.new_pos = -1;
            int rc = is_quant(kc->fmt) ? launch_sdpa_decode_quant(a, s) : launch_sdpa_decode(a, s);
            if (rc == 0) {
                kc->len += 1;
                vc->len += 1;
                return 0;
            }
            if (rc != 2) return rc;
        }
    }
    if (trocm_kv_append_pair(kc, vc, k_new, v_new, dtype, kv_new_strides, n_new, stream)) return 1;
    return trocm_sdpa_cached(q, dtype, q_heads, n_new, kc, vc, out, scale, causal, workspace, workspace_bytes, stream);
}

// ApplyRope on q and k_new, then InPlaceKvSdpaState::eval: what an exported decoder's graph does with the two ApplyRope
// nodes between the projections and the cache.  A single-token step on an f16 cache is ONE launch (the attention
// kernel rotates both on the way in); every other call rotates into `rot_scratch` and goes on as trocm_inplace_kv_sdpa_eval.
int trocm_inplace_kv_sdpa_eval_rope(const void *q, const void *k_new, const void *v_new, const void *cos, const void *sin,
                                    int64_t cos_sin_batch_stride, int dtype, int64_t q_heads, int64_t n_new,
                                    trocm_kv_cache *kc, trocm_kv_cache *vc, void *out, float scale, int causal,
                                    void *workspace, size_t workspace_bytes, void *rot_scratch, size_t rot_scratch_bytes,
                                    void *stream) {
    if (inplace_eval_check("inplace_kv_sdpa_rope", q, k_new, v_new, out, dtype, q_heads, n_new, kc, vc)) return 1;
    TROCM_NOT_NULL(cos);
    TROCM_NOT_NULL(sin);
    TROCM_REQUIRE(kc->D % 2 == 0, "apply_rope: the head dimension must be even");
    TROCM_REQUIRE(cos_sin_batch_stride == 0 || cos_sin_batch_stride >= n_new * kc->D,
                  "apply_rope: cos / sin rows of one sequence overlap the next one's (batch stride %lld < %lld)",
                  (long long)cos_sin_batch_stride, (long long)(n_new * kc->D));
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    if (n_new == 1 && dtype == TROCM_F16 && (kc->fmt == TROCM_F16 || is_quant(kc->fmt)) && kc->window == 0 && vc->window == 0 && q_heads % kc->H == 0) {
        if (equalise_capacities(kc, vc, s)) return 1;
        int64_t dense[4];
        dense[3] = 1, dense[2] = kc->D, dense[1] = kc->D, dense[0] = kc->H * kc->D;
        if (append_prepare(kc, k_new, dtype, dense, 1, s)) return 1;
        if (append_prepare(vc, v_new, dtype, dense, 1, s)) return 1;
        if (kc->cap == vc->cap) {
            SdpaArgs a;
            cached_args(a, q, dtype, q_heads, 1, kc, vc, kc->len + 1, out, scale, causal, workspace, workspace_bytes);
            a.k_new = k_new, a.v_new = v_new, a.new_pos = -1;
            a.rope_cos = cos, a.rope_sin = sin, a.rope_stride_b = cos_sin_batch_stride;
            int rc = is_quant(kc->fmt) ? launch_sdpa_decode_quant(a, s) : launch_sdpa_decode(a, s);
            if (rc == 0) {
                kc->len += 1;
                vc->len += 1;
                return 0;
            }
            if (rc != 2) return rc;
        }
    }
    // rotate into the caller's scratch: q first, then k_new
    const size_t es = elem_bytes(dtype);
    const size_t q_bytes = (size_t)kc->B * q_heads * n_new * kc->D * es, k_bytes = (size_t)kc->B * kc->H * n_new * kc->D * es;
    const size_t q_room = (q_bytes + 255) & ~(size_t)255;
    TROCM_REQUIRE(rot_scratch != nullptr && rot_scratch_bytes >= q_room + k_bytes,
                  "inplace_kv_sdpa_rope: this call rotates q and k_new into rot_scratch, which must hold %zu bytes (%zu given)",
                  q_room + k_bytes, rot_scratch_bytes);
    TROCM_REQUIRE((uintptr_t)rot_scratch % 16 == 0, "rot_scratch must be 16-byte aligned");
    void *q_rot = rot_scratch, *k_rot = (char *)rot_scratch + q_room;
    const int64_t cs[4] = {cos_sin_batch_stride, 0, kc->D, 1};
    const int64_t qs[4] = {kc->B, q_heads, n_new, kc->D}, ks[4] = {kc->B, kc->H, n_new, kc->D};
    if (n_new > 0) {
        if (trocm_apply_rope(q, cos, sin, q_rot, dtype, 4, qs, nullptr, cs, nullptr, stream)) return 1;
        if (trocm_apply_rope(k_new, cos, sin, k_rot, dtype, 4, ks, nullptr, cs, nullptr, stream)) return 1;
    }
    return trocm_inplace_kv_sdpa_eval(q_rot, k_rot, v_new, dtype, q_heads, n_new, nullptr, kc, vc, out, scale, causal, workspace,
                                      workspace_bytes, stream);
}

// WindowKvSdpaState::eval (window_kv_cache.rs:216-239): push K_new / V_new into the ring buffers,
// then attend to every valid slot in physical order without a causal mask -- the ring buffer
// already bounds which keys are visible, and attention does not depend on the order of the keys.
int trocm_window_kv_sdpa_eval(const void *q, const void *k_new, const void *v_new, int dtype, int64_t q_heads,
                              int64_t n_new, const int64_t *kv_new_strides, trocm_kv_cache *kc, trocm_kv_cache *vc,
                              void *out, float scale, void *workspace, size_t workspace_bytes, void *stream) {
    TROCM_NOT_NULL(kc);
    TROCM_NOT_NULL(vc);
    TROCM_REQUIRE(kc->window > 0 && vc->window == kc->window, "window_kv_sdpa: K and V must be sliding-window caches of one window");
    if (inplace_eval_check("window_kv_sdpa", q, k_new, v_new, out, dtype, q_heads, n_new, kc, vc)) return 1;
    TROCM_REQUIRE(kc->cursor == vc->cursor, "K and V ring cursors must match");
    if (kv_new_strides)
        for (int i = 0; i < 4; i++) TROCM_REQUIRE(kv_new_strides[i] >= 0, "append: negative source strides are not supported");
    int64_t dense[4];
    dense[3] = 1, dense[2] = kc->D, dense[1] = n_new * kc->D, dense[0] = kc->H * n_new * kc->D;
    bool is_dense = kv_new_strides == nullptr;
    if (!is_dense) {
        is_dense = true;
        for (int i = 0; i < 4; i++) is_dense = is_dense && kv_new_strides[i] == dense[i];
    } else {
        kv_new_strides = dense;
    }
    // Decode step on a plain-format ring: the attention kernel reads the new token from the inputs and
    // stores it at the cursor itself -- one launch instead of append + attention.
    if (n_new == 1 && is_dense && !is_quant(kc->fmt) && dtype == kc->fmt && q && k_new && v_new && out && kc->fmt == vc->fmt &&
        kc->B == vc->B && kc->H == vc->H && kc->D == vc->D && kc->len == vc->len && kc->cursor == vc->cursor &&
        q_heads % kc->H == 0) {
        hipStream_t s;
        if (resolve_stream(stream, &s)) return 1;
        if (append_prepare(kc, k_new, dtype, kv_new_strides, 1, s)) return 1;
        if (append_prepare(vc, v_new, dtype, kv_new_strides, 1, s)) return 1;
        if (kc->cap == vc->cap && kc->cap == kc->window) {
            const int64_t w = kc->window, new_len = kc->len + 1 < w ? kc->len + 1 : w;
            SdpaArgs a;
            cached_args(a, q, dtype, q_heads, 1, kc, vc, new_len, out, scale, 0, workspace, workspace_bytes);
            a.k_new = k_new, a.v_new = v_new, a.new_pos = kc->cursor;
            int rc = launch_sdpa_decode(a, s);
            if (rc == 0) {
                kc->cursor = vc->cursor = kc->cursor + 1 == w ? 0 : kc->cursor + 1;
                kc->len = vc->len = new_len;
                return 0;
            }
            if (rc != 2) return rc;
        }
    }
    if (trocm_kv_append_pair(kc, vc, k_new, v_new, dtype, kv_new_strides, n_new, stream)) return 1;
    return trocm_sdpa_cached(q, dtype, q_heads, n_new, kc, vc, out, scale, 0, workspace, workspace_bytes, stream);
}

static int ragged_common(const void *q, const void *k_new, const void *v_new, int q_dtype, int64_t q_heads,
                         int64_t n_seq, trocm_kv_cache *const *k_caches, trocm_kv_cache *const *v_caches, void *out,
                         float scale, void *workspace, size_t workspace_bytes, void *stream, const void *rope_cos = nullptr,
                         const void *rope_sin = nullptr, void *rot_scratch = nullptr, size_t rot_scratch_bytes = 0) {
    TROCM_NOT_NULL(q);
    TROCM_NOT_NULL(k_caches);
    TROCM_NOT_NULL(v_caches);
    TROCM_NOT_NULL(out);
    TROCM_REQUIRE(n_seq >= 1, "ragged decode: n_seq must be >= 1");
    hipStream_t s;
    if (resolve_stream(stream, &s)) return 1;
    const bool fused = k_new != nullptr;
    if (fused) TROCM_NOT_NULL(v_new);
    std::vector<RaggedSeq> seqs((size_t)n_seq);
    trocm_kv_cache *k0 = k_caches[0];
    TROCM_NOT_NULL(k0);
    for (int64_t i = 0; i < n_seq; i++) {
        trocm_kv_cache *kc = k_caches[i], *vc = v_caches[i];
        TROCM_NOT_NULL(kc);
        TROCM_NOT_NULL(vc);
        TROCM_REQUIRE(kc->B == 1 && vc->B == 1, "ragged decode: every per-sequence cache must have batch == 1");
        TROCM_REQUIRE(kc->fmt == k0->fmt && vc->fmt == k0->fmt && kc->H == k0->H && vc->H == k0->H && kc->D == k0->D &&
                          vc->D == k0->D,
                      "ragged decode: caches differ in format or shape (sequence %lld)", (long long)i);
        TROCM_REQUIRE(kc->len == vc->len, "K/V lengths must match (sequence %lld)", (long long)i);
        TROCM_REQUIRE(!fused || (kc->window == 0 && vc->window == 0),
                      "ragged fused step: sliding-window caches are not supported (sequence %lld)", (long long)i);
    }
    TROCM_REQUIRE(q_heads % k0->H == 0, "Q heads (%lld) must be a multiple of K/V heads (%lld)", (long long)q_heads,
                  (long long)k0->H);
    TROCM_REQUIRE(is_quant(k0->fmt) || k0->fmt == q_dtype, "q dtype %d does not match the cache format %d", q_dtype,
                  k0->fmt);
    const int64_t row_elems = k0->H * k0->D;  // one sequence's new token, all kv heads
    const size_t es = elem_bytes(q_dtype);
    int64_t dense[4] = {row_elems, k0->D, k0->D, 1};
    bool in_kernel = fused && (!is_quant(k0->fmt) || q_dtype == TROCM_F16);   // (quantised caches: f16 rows, quantised by the attention kernel)
    // RoPE on q and k_new: inside the attention launch where a kernel does it, else into the caller's scratch first
    const size_t rot_q_room = ((size_t)n_seq * q_heads * k0->D * es + 255) & ~(size_t)255;
    const size_t rot_need = rot_q_room + (size_t)n_seq * row_elems * es;
    auto rotate_into_scratch = [&]() -> int {
        void *q_rot = rot_scratch, *k_rot = (char *)rot_scratch + rot_q_room;
        const int64_t cs[4] = {k0->D, 0, k0->D, 1};
        const int64_t qs[4] = {n_seq, q_heads, 1, k0->D}, ks[4] = {n_seq, k0->H, 1, k0->D};
        if (trocm_apply_rope(q, rope_cos, rope_sin, q_rot, q_dtype, 4, qs, nullptr, cs, nullptr, stream)) return 1;
        if (trocm_apply_rope(k_new, rope_cos, rope_sin, k_rot, q_dtype, 4, ks, nullptr, cs, nullptr, stream)) return 1;
        q = q_rot, k_new = k_rot, rope_cos = rope_sin = nullptr;
        return 0;
    };
    if (rope_cos) {
        TROCM_REQUIRE(fused && rope_sin, "RoPE is folded into the step that appends (k_new, v_new, cos and sin)");
        TROCM_REQUIRE(k0->D % 2 == 0, "apply_rope: the head dimension must be even");
        // Whether a kernel takes the rotation is known when the launcher answers, after the caches may have grown: a call
        // that could need the scratch and has none is refused here, before anything is changed.
        const bool kernel_rotates = in_kernel && q_dtype == TROCM_F16 && q_heads % k0->H == 0 && q_heads / k0->H >= 2 &&
                                    (k0->fmt == TROCM_F16 ? q_heads / k0->H <= 16 && (k0->D == 64 || k0->D == 128)
                                                          : is_quant(k0->fmt) && decode_quant_rotates_in_kernel(q_heads / k0->H));
        if (!kernel_rotates) {
            TROCM_REQUIRE(rot_scratch != nullptr && rot_scratch_bytes >= rot_need && (uintptr_t)rot_scratch % 16 == 0,
                          "ragged step with RoPE: this call rotates q and k_new into rot_scratch, which must be 16-byte aligned and hold %zu bytes (%zu given)",
                          rot_need, rot_scratch_bytes);
            if (rotate_into_scratch()) return 1;
        }
    }
    if (fused) {  // growth first (may reallocate), for every sequence
        for (int64_t i = 0; i < n_seq; i++) {
            const char *kn = (const char *)k_new + (size_t)i * row_elems * es, *vn = (const char *)v_new + (size_t)i * row_elems * es;
            if (append_prepare(k_caches[i], kn, q_dtype, dense, 1, s)) return 1;
            if (append_prepare(v_caches[i], vn, q_dtype, dense, 1, s)) return 1;
        }
    }
    float sc = isnan(scale) ? 1.0f / sqrtf((float)k0->D) : scale;
    auto append_explicitly = [&]() -> int {
        for (int64_t i = 0; i < n_seq; i++) {
            const char *kn = (const char *)k_new + (size_t)i * row_elems * es, *vn = (const char *)v_new + (size_t)i * row_elems * es;
            if (append_write(k_caches[i], kn, q_dtype, dense, 1, s)) return 1;
            if (append_write(v_caches[i], vn, q_dtype, dense, 1, s)) return 1;
            k_caches[i]->len += 1, v_caches[i]->len += 1;
        }
        return 0;
    };
    // Quantised caches: one launch quantises every sequence's new token (its table travels in the plan area of
    // the workspace, which the attention launch rewrites afterwards, in stream order).
    auto append_quantised_at_once = [&]() -> int {
        std::vector<QuantAppendSeq> tbl((size_t)n_seq);
        for (int64_t i = 0; i < n_seq; i++) {
            trocm_kv_cache *kc = k_caches[i], *vc = v_caches[i];
            TROCM_REQUIRE(kc->pitch == vc->pitch, "K/V capacities must match (sequence %lld)", (long long)i);
            tbl[(size_t)i] = QuantAppendSeq{kc->data, kc->scales, vc->data, vc->scales, kc->pitch, kc->len};
        }
        void *dev_tbl = (char *)workspace + kWsCounterBytes;
        if (upload_table(tbl.data(), tbl.size() * sizeof(QuantAppendSeq), dev_tbl, s)) return 1;
        if (launch_quant_append_ragged(k0->fmt, q_dtype, n_seq, k0->H, k0->D, (const QuantAppendSeq *)dev_tbl, k_new, v_new, s)) return 1;
        for (int64_t i = 0; i < n_seq; i++) k_caches[i]->len += 1, v_caches[i]->len += 1;
        return 0;
    };
    if (fused && !in_kernel) {
        const bool at_once = is_quant(k0->fmt) && workspace != nullptr && workspace_bytes >= kWsCounterBytes + kWsPlanBytes &&
                             (size_t)n_seq * sizeof(QuantAppendSeq) <= kWsPlanBytes && k0->D % 32 == 0;
        if (at_once ? append_quantised_at_once() : append_explicitly()) return 1;
    }
    for (;;) {
        for (int64_t i = 0; i < n_seq; i++) {
            const trocm_kv_cache *kc = k_caches[i], *vc = v_caches[i];
            TROCM_REQUIRE(kc->cap == vc->cap, "K/V capacities must match (sequence %lld)", (long long)i);
            int64_t len = kc->len + (in_kernel ? 1 : 0);
            TROCM_REQUIRE(len > 0, "empty kv-cache (sequence %lld)", (long long)i);
            seqs[(size_t)i] = RaggedSeq{kc->data, vc->data, kc->scales, vc->scales, len, kc->pitch};
        }
        int rc = launch_sdpa_decode_ragged(q, out, q_dtype, k0->fmt, n_seq, q_heads, k0->H, k0->D, seqs.data(), sc,
                                           workspace, workspace_bytes, in_kernel ? k_new : nullptr,
                                           in_kernel ? v_new : nullptr, s, in_kernel ? rope_cos : nullptr, in_kernel ? rope_sin : nullptr);
        if (rc == 0 && in_kernel)
            for (int64_t i = 0; i < n_seq; i++) k_caches[i]->len += 1, v_caches[i]->len += 1;
        if (rc != 2) return rc;
        if (!in_kernel) return fail("ragged decode: no kernel covers this shape");
        if (rope_cos) {   // (alignment, a workspace too small ...) no kernel rotates after all: rotate first if there is room, then go on
            if (rot_scratch == nullptr || rot_scratch_bytes < rot_need || (uintptr_t)rot_scratch % 16)
                return fail("ragged step with RoPE: no kernel rotates for this call and rot_scratch does not hold %zu bytes", rot_need);
            if (rotate_into_scratch()) return 1;
            continue;
        }
        // the kernel cannot append in place for this shape: append explicitly, then attend
        in_kernel = false;
        const bool at_once = is_quant(k0->fmt) && workspace != nullptr && workspace_bytes >= kWsCounterBytes + kWsPlanBytes &&
                             (size_t)n_seq * sizeof(QuantAppendSeq) <= kWsPlanBytes && k0->D % 32 == 0;
        if (at_once ? append_quantised_at_once() : append_explicitly()) return 1;
    }
}

int trocm_sdpa_decode_ragged(const void *q, int q_dtype, int64_t q_heads, int64_t n_seq,
                             trocm_kv_cache *const *k_caches, trocm_kv_cache *const *v_caches, void *out, float scale,
                             void *workspace, size_t workspace_bytes, void *stream) {
    return ragged_common(q, nullptr, nullptr, q_dtype, q_heads, n_seq, k_caches, v_caches, out, scale, workspace,
                         workspace_bytes, stream);
}

int trocm_inplace_kv_sdpa_eval_ragged(const void *q, const void *k_new, const void *v_new, int dtype, int64_t q_heads,
                                      int64_t n_seq, trocm_kv_cache *const *k_caches, trocm_kv_cache *const *v_caches,
                                      void *out, float scale, void *workspace, size_t workspace_bytes, void *stream) {
    TROCM_NOT_NULL(k_new);
    TROCM_NOT_NULL(v_new);
    return ragged_common(q, k_new, v_new, dtype, q_heads, n_seq, k_caches, v_caches, out, scale, workspace,
                         workspace_bytes, stream);
}

// The ragged step with its RoPE folded in: cos and sin are [n_seq, head_dim] rows of `dtype` (each sequence's position).
int trocm_inplace_kv_sdpa_eval_ragged_rope(const void *q, const void *k_new, const void *v_new, const void *cos, const void *sin,
                                           int dtype, int64_t q_heads, int64_t n_seq, trocm_kv_cache *const *k_caches,
                                           trocm_kv_cache *const *v_caches, void *out, float scale, void *workspace,
                                           size_t workspace_bytes, void *rot_scratch, size_t rot_scratch_bytes, void *stream) {
    TROCM_NOT_NULL(k_new);
    TROCM_NOT_NULL(v_new);
    TROCM_NOT_NULL(cos);
    TROCM_NOT_NULL(sin);
    return ragged_common(q, k_new, v_new, dtype, q_heads, n_seq, k_caches, v_caches, out, scale, workspace, workspace_bytes,
                         stream, cos, sin, rot_scratch, rot_scratch_bytes);
}

}  // extern "C"
