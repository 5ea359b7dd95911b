// Context, memory, error and profiler plumbing of libskm_hip.so.
#include "skm_internal.h"

#include <cstdlib>

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <mutex>
#include <thread>
#include <unordered_map>

namespace skm {

static thread_local char g_last_error[512] = "";

int set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return SKM_OK;
    const int code = (e == hipErrorOutOfMemory) ? SKM_ERR_OOM : SKM_ERR_HIP;
    return set_error(code, "HIP error %d (%s) in %s", (int) e, hipGetErrorString(e), what);
}

// ---------------------------------------------------------------------------------------------
// Device blocks released by skm_free, by a context's workspace or by skm_ctx_destroy are kept and handed out
// again: hipMalloc / hipFree of the gigabyte-sized buffers of a Train cost milliseconds each and hipFree waits
// for the whole device.  One cache per device and process; a request takes the smallest cached block of at least
// its size and at most 1/8 more.  The cache holds at most its byte limit and DEVICE_CACHE_MAX_BLOCKS
// (beyond that a released block goes back to the driver), and is emptied when an allocation fails or on
// skm_device_cache_trim.  A block enters the cache only after the releasing context's stream has drained.
// ---------------------------------------------------------------------------------------------
namespace {
constexpr size_t DEVICE_CACHE_DEFAULT_MAX_BYTES = size_t(48) << 30;
constexpr size_t DEVICE_CACHE_MAX_BLOCKS = 2048;
// Limit of the idle bytes: SKM_DEVICE_CACHE_BYTES in the environment when the process first uses a device, else the
// default; skm_device_cache_set_limit changes it later.
static size_t initial_cache_limit() {
    const char* env = getenv("SKM_DEVICE_CACHE_BYTES");
    if (env && *env) {
        char* end = nullptr;
        const unsigned long long v = strtoull(env, &end, 10);
        if (end && *end == '\0') return (size_t) v;
    }
    return DEVICE_CACHE_DEFAULT_MAX_BYTES;
}
struct DeviceCache {
    std::mutex lock;
    size_t max_bytes = initial_cache_limit();
    std::multimap<size_t, void*> idle;           // size -> block
    std::unordered_map<void*, size_t> size_of;   // every block handed out or idle
    size_t idle_bytes = 0;
};
DeviceCache& device_cache(int device) {
    static DeviceCache caches[64];
    return caches[(device >= 0 && device < 64) ? device : 0];
}
void trim_locked(DeviceCache& c) {
    for (auto& kv : c.idle) {
        (void) hipFree(kv.second);
        c.size_of.erase(kv.second);
    }
    c.idle.clear();
    c.idle_bytes = 0;
}
} // namespace

int device_alloc(int device, size_t bytes, void** out) {
    *out = nullptr;
    if (bytes == 0) bytes = 16;
    bytes = (bytes + 255) / 256 * 256;
    DeviceCache& c = device_cache(device);
    std::lock_guard<std::mutex> guard(c.lock);
    auto it = c.idle.lower_bound(bytes);
    if (it != c.idle.end() && it->first <= bytes + bytes / 8) {
        *out = it->second;
        c.idle_bytes -= it->first;
        c.idle.erase(it);
        return SKM_OK;
    }
    hipError_t e = hipMalloc(out, bytes);
    if (e != hipSuccess) {
        (void) hipGetLastError();
        trim_locked(c);
        e = hipMalloc(out, bytes);
    }
    if (e != hipSuccess) return check_hip(e, "hipMalloc");
    c.size_of[*out] = bytes;
    return SKM_OK;
}

// The caller guarantees that no queued work uses the block any more.
int device_release(int device, void* ptr) {
    if (!ptr) return SKM_OK;
    DeviceCache& c = device_cache(device);
    std::lock_guard<std::mutex> guard(c.lock);
    const auto known = c.size_of.find(ptr);
    if (known == c.size_of.end()) return check_hip(hipFree(ptr), "hipFree");  // not one of ours
    const size_t bytes = known->second;
    if (c.idle.size() >= DEVICE_CACHE_MAX_BLOCKS || c.idle_bytes + bytes > c.max_bytes) {
        c.size_of.erase(known);
        return check_hip(hipFree(ptr), "hipFree");
    }
    c.idle.emplace(bytes, ptr);
    c.idle_bytes += bytes;
    return SKM_OK;
}

int workspace(skm_ctx* ctx, int slot, size_t bytes, void** out) {
    if (slot < 0 || slot >= skm_ctx::WS_SLOTS) return set_error(SKM_ERR_INVALID, "bad workspace slot");
    if (ctx->ws_bytes[slot] < bytes) {
        if (ctx->ws[slot]) {
            // a slot that grows again gets a quarter more than it held: requests that creep up call after call (the
            // dense rows of the overflowing points of one slab after another) would otherwise reallocate every time
            // (within the workspace limit, unless the request itself is beyond it)
            size_t roomy = ctx->ws_bytes[slot] + ctx->ws_bytes[slot] / 4;
            if (roomy > ctx->workspace_limit) roomy = ctx->workspace_limit;
            if (bytes < roomy) bytes = roomy;
            SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
            SKM_TRY(device_release(ctx->device, ctx->ws[slot]));
            ctx->ws[slot] = nullptr;
            ctx->ws_bytes[slot] = 0;
            if (slot == 4) {
                ctx->cluster_order = nullptr;
                ctx->cluster_order_n = 0;
            }
        }
        SKM_TRY(device_alloc(ctx->device, bytes, &ctx->ws[slot]));
        ctx->ws_bytes[slot] = bytes;
    }
    *out = ctx->ws[slot];
    return SKM_OK;
}

// One pinned host block per context, allocated at first use (pinned allocations are slow and every helper context of
// a hierarchical Train has its own): result slots, then the copy of the cluster sizes, then the ring of row edits.
constexpr size_t PINNED_SLOTS_BYTES = 256;
constexpr size_t PINNED_SIZES_BYTES = size_t(16384) * sizeof(uint32_t);
constexpr size_t PINNED_RING_BYTES = size_t(256) << 10;

static int pinned_block(skm_ctx* ctx) {
    if (!ctx->h_pinned) {
        const size_t total = PINNED_SLOTS_BYTES + PINNED_SIZES_BYTES + PINNED_RING_BYTES;
        SKM_HIP_TRY(hipHostMalloc(&ctx->h_pinned, total, hipHostMallocDefault));
        ctx->h_pinned_bytes = total;
        ctx->h_ring_used = 0;
    }
    return SKM_OK;
}

int pinned(skm_ctx* ctx, size_t bytes, void** out) {
    if (bytes > PINNED_SLOTS_BYTES) return set_error(SKM_ERR_INVALID, "pinned: %zu bytes of result slots requested", bytes);
    SKM_TRY(pinned_block(ctx));
    *out = ctx->h_pinned;
    return SKM_OK;
}

int pinned_sizes(skm_ctx* ctx, uint32_t** out, size_t* out_entries) {
    SKM_TRY(pinned_block(ctx));
    *out = reinterpret_cast<uint32_t*>((char*) ctx->h_pinned + PINNED_SLOTS_BYTES);
    *out_entries = PINNED_SIZES_BYTES / sizeof(uint32_t);
    return SKM_OK;
}

int host_ring(skm_ctx* ctx, void** out, size_t* out_bytes) {
    SKM_TRY(pinned_block(ctx));
    *out = (char*) ctx->h_pinned + PINNED_SLOTS_BYTES + PINNED_SIZES_BYTES;
    *out_bytes = PINNED_RING_BYTES;
    return SKM_OK;
}

int reduction_counter(skm_ctx* ctx, uint32_t** out) {
    if (!ctx->d_reduction_counter) {
        void* p = nullptr;
        SKM_TRY(device_alloc(ctx->device, 256, &p));
        const hipError_t e = hipMemsetAsync(p, 0, 256, ctx->stream);
        if (e != hipSuccess) {
            (void) device_release(ctx->device, p);
            return check_hip(e, "hipMemsetAsync");
        }
        ctx->d_reduction_counter = (uint32_t*) p;
    }
    *out = ctx->d_reduction_counter;
    return SKM_OK;
}

static hipEvent_t take_event(skm_ctx* ctx) {
    if (!ctx->event_pool.empty()) {
        hipEvent_t e = ctx->event_pool.back();
        ctx->event_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}

ScopedStage::ScopedStage(skm_ctx* ctx, const char* scope) : ctx_(ctx) {
    if (!ctx->prof) return;
    iv_.scope = scope;
    iv_.start = take_event(ctx);
    iv_.stop = take_event(ctx);
    if (!iv_.start || !iv_.stop) return;
    if (hipEventRecord(iv_.start, ctx->stream) != hipSuccess) return;
    active_ = true;
}

ScopedStage::~ScopedStage() {
    if (!active_) return;
    if (hipEventRecord(iv_.stop, ctx_->stream) != hipSuccess) return;
    ctx_->pending.push_back(iv_);
    if (ctx_->pending.size() >= 4096) resolve_pending(ctx_);
}

int resolve_pending(skm_ctx* ctx) {
    if (ctx->pending.empty()) return SKM_OK;
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    for (auto& iv : ctx->pending) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, iv.start, iv.stop) == hipSuccess) {
            auto& t = ctx->timers[iv.scope];
            t.ms += ms;
            t.calls += 1;
        }
        ctx->event_pool.push_back(iv.start);
        ctx->event_pool.push_back(iv.stop);
    }
    ctx->pending.clear();
    return SKM_OK;
}

__global__ void fill_u32_kernel(uint32_t* dst, uint32_t value, size_t count) {
    size_t i = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t) gridDim.x * blockDim.x;
    for (; i < count; i += stride) dst[i] = value;
}

} // namespace skm

using namespace skm;

extern "C" {

const char* skm_last_error(void) { return g_last_error; }

int skm_device_count(int* out_count) {
    if (!out_count) return set_error(SKM_ERR_INVALID, "skm_device_count: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *out_count = 0;
        return set_error(SKM_ERR_NO_DEVICE, "no HIP device: %s", hipGetErrorString(e));
    }
    *out_count = n;
    return SKM_OK;
}

int skm_ctx_create(int device, skm_ctx** out_ctx) {
    if (!out_ctx) return set_error(SKM_ERR_INVALID, "skm_ctx_create: null output");
    *out_ctx = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0)
        return set_error(SKM_ERR_NO_DEVICE, "skm_ctx_create: no HIP device is visible");
    if (device < 0 || device >= n)
        return set_error(SKM_ERR_INVALID, "skm_ctx_create: device %d out of range [0,%d)", device, n);
    SKM_HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    SKM_HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(SKM_ERR_NO_DEVICE, "skm_ctx_create: device %d is %s; this library is built for gfx950 only",
                         device, prop.gcnArchName);
    void* noalloc_scratch = nullptr;
    SKM_TRY(resolve_noalloc_scratch(device, &noalloc_scratch));
    skm_ctx* ctx = new skm_ctx();
    ctx->device = device;
    ctx->noalloc_scratch = noalloc_scratch;
    hipError_t e = hipStreamCreate(&ctx->stream);
    if (e != hipSuccess) {
        delete ctx;
        return check_hip(e, "hipStreamCreate");
    }
    // The pinned block is made here rather than at its first use, which falls into the middle of an iteration:
    // pinning host memory while kernels run holds them up (helper contexts are created while the device is idle).
    const int rc = pinned_block(ctx);
    if (rc != SKM_OK) {
        (void) hipStreamDestroy(ctx->stream);
        delete ctx;
        return rc;
    }
    *out_ctx = ctx;
    return SKM_OK;
}

int skm_ctx_destroy(skm_ctx* ctx) {
    if (!ctx) return SKM_OK;
    // Teardown keeps going after a failure so that every resource gets its release call.
    (void) hipSetDevice(ctx->device);
    (void) hipStreamSynchronize(ctx->stream);
    for (auto& iv : ctx->pending) {
        (void) hipEventDestroy(iv.start);
        (void) hipEventDestroy(iv.stop);
    }
    for (auto e : ctx->event_pool) (void) hipEventDestroy(e);
    for (int i = 0; i < skm_ctx::WS_SLOTS; ++i)
        if (ctx->ws[i]) (void) device_release(ctx->device, ctx->ws[i]);
    if (ctx->d_reduction_counter) (void) device_release(ctx->device, ctx->d_reduction_counter);
    if (ctx->h_pinned) (void) hipHostFree(ctx->h_pinned);
    for (auto s : ctx->download_stream)
        if (s) (void) hipStreamDestroy(s);
    if (ctx->download_staging) (void) hipHostFree(ctx->download_staging);
    if (ctx->copy_stream) {
        (void) hipStreamSynchronize(ctx->copy_stream);
        for (auto e : ctx->copy_done)
            if (e) (void) hipEventDestroy(e);
        (void) hipStreamDestroy(ctx->copy_stream);
    }
    (void) hipStreamDestroy(ctx->stream);
    delete ctx;
    return SKM_OK;
}

int skm_sync(skm_ctx* ctx) {
    SKM_REQUIRE(ctx, "null context");
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SKM_OK;
}

int skm_ctx_set_workspace_limit(skm_ctx* ctx, size_t bytes) {
    SKM_REQUIRE(ctx, "null context");
    SKM_REQUIRE(bytes >= (size_t(64) << 20), "workspace limit must be at least 64 MiB");
    ctx->workspace_limit = bytes;
    return SKM_OK;
}

int skm_ctx_set_candidate_kernel(skm_ctx* ctx, int which) {
    SKM_REQUIRE(ctx, "null context");
    SKM_REQUIRE(which >= 0 && which <= 3, "which must be 0 (automatic), 1 (tiled), 2 (register-stationary) or 3 (large tiles)");
    ctx->candidate_kernel = which;
    return SKM_OK;
}

int skm_ctx_set_walk_kernel(skm_ctx* ctx, int which) {
    SKM_REQUIRE(ctx, "null context");
    SKM_REQUIRE(which >= 0 && which <= 3, "which must be 0 (automatic), 1 (one point per wavefront), 2 or 3 (pooled, 4 or 8 points)");
    ctx->walk_kernel = which;
    return SKM_OK;
}

int skm_ctx_get_last_overflow(skm_ctx* ctx, uint64_t* out_points) {
    SKM_REQUIRE(ctx && out_points, "null argument");
    *out_points = ctx->last_overflow_points;
    return SKM_OK;
}

int skm_ctx_set_walk_launches(skm_ctx* ctx, int launches) {
    SKM_REQUIRE(ctx, "null context");
    SKM_REQUIRE(launches >= 1, "launches must be at least 1");
    ctx->walk_launches = launches;
    return SKM_OK;
}

int skm_malloc(skm_ctx* ctx, size_t bytes, void** out_d_ptr) {
    SKM_REQUIRE(ctx && out_d_ptr, "null argument");
    SKM_HIP_TRY(hipSetDevice(ctx->device));
    return device_alloc(ctx->device, bytes, out_d_ptr);
}

int skm_device_cache_set_limit(int device, size_t bytes) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n)
        return set_error(SKM_ERR_INVALID, "skm_device_cache_set_limit: no such device");
    SKM_HIP_TRY(hipSetDevice(device));
    DeviceCache& c = device_cache(device);
    std::lock_guard<std::mutex> guard(c.lock);
    c.max_bytes = bytes;
    if (c.idle_bytes > bytes) trim_locked(c);
    return SKM_OK;
}

int skm_device_cache_trim(int device) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device < 0 || device >= n)
        return set_error(SKM_ERR_INVALID, "skm_device_cache_trim: no such device");
    SKM_HIP_TRY(hipSetDevice(device));
    DeviceCache& c = device_cache(device);
    std::lock_guard<std::mutex> guard(c.lock);
    trim_locked(c);
    return SKM_OK;
}

int skm_free(skm_ctx* ctx, void* d_ptr) {
    SKM_REQUIRE(ctx, "null context");
    if (!d_ptr) return SKM_OK;
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (ctx->copy_stream) SKM_HIP_TRY(hipStreamSynchronize(ctx->copy_stream));
    return device_release(ctx->device, d_ptr);
}

int skm_upload(skm_ctx* ctx, void* d_dst, const void* h_src, size_t bytes) {
    SKM_REQUIRE(ctx, "null context");
    if (bytes == 0) return SKM_OK;
    SKM_REQUIRE(d_dst && h_src, "null pointer");
    SKM_HIP_TRY(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->stream));
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SKM_OK;
}

namespace {
// The transfer stream of a context and the events that order it before the context's stream, made on first use.
int ensure_copy_stream(skm_ctx* ctx) {
    if (ctx->copy_stream) return SKM_OK;
    hipStream_t s = nullptr;
    SKM_HIP_TRY(hipStreamCreate(&s));
    for (auto& e : ctx->copy_done) {
        const hipError_t rc = hipEventCreateWithFlags(&e, hipEventDisableTiming);
        if (rc != hipSuccess) {
            for (auto& made : ctx->copy_done) {
                if (made) (void) hipEventDestroy(made);
                made = nullptr;
            }
            (void) hipStreamDestroy(s);
            return check_hip(rc, "hipEventCreateWithFlags");
        }
    }
    ctx->copy_stream = s;
    return SKM_OK;
}
} // namespace

int skm_upload_overlapped(skm_ctx* ctx, void* d_dst, const void* h_src, size_t bytes) {
    SKM_REQUIRE(ctx, "null context");
    if (bytes == 0) return SKM_OK;
    SKM_REQUIRE(d_dst && h_src, "null pointer");
    SKM_HIP_TRY(hipSetDevice(ctx->device));
    SKM_TRY(ensure_copy_stream(ctx));
    hipEvent_t done = ctx->copy_done[ctx->copy_seq++ % 8];
    SKM_HIP_TRY(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->copy_stream));
    SKM_HIP_TRY(hipEventRecord(done, ctx->copy_stream));
    SKM_HIP_TRY(hipStreamWaitEvent(ctx->stream, done, 0));
    return SKM_OK;
}

int skm_upload_detached(skm_ctx* ctx, void* d_dst, const void* h_src, size_t bytes) {
    SKM_REQUIRE(ctx, "null context");
    SKM_HIP_TRY(hipSetDevice(ctx->device));
    SKM_TRY(ensure_copy_stream(ctx));  // also for zero bytes: the owner's way to make the stream before a feeder starts
    if (bytes == 0) return SKM_OK;
    SKM_REQUIRE(d_dst && h_src, "null pointer");
    SKM_HIP_TRY(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, ctx->copy_stream));
    SKM_HIP_TRY(hipStreamSynchronize(ctx->copy_stream));
    return SKM_OK;
}

// A copy from the device into pageable host memory goes through a pinned staging block: a transfer into the block,
// then a copy by the processor to the destination.  The runtime does the two steps one after the other on one
// thread, which gives about 10 GB/s; here DOWNLOAD_LANES threads each take every DOWNLOAD_LANES-th chunk, so the
// transfers of some overlap the processor copies of the others (the 268 MB of 65,536 centroids of 1,024 dimensions:
// 28 ms through the runtime).  Used from DOWNLOAD_LANES_MIN_BYTES, where it repays the threads and, the first time,
// the staging blocks.
namespace {
constexpr size_t DOWNLOAD_CHUNK = size_t(4) << 20;
constexpr size_t DOWNLOAD_LANES_MIN_BYTES = size_t(64) << 20;

int download_in_lanes(skm_ctx* ctx, char* h_dst, const char* d_src, size_t bytes) {
    constexpr int LANES = skm_ctx::DOWNLOAD_LANES;
    SKM_HIP_TRY(hipSetDevice(ctx->device));
    if (!ctx->download_staging) {
        void* block = nullptr;
        SKM_HIP_TRY(hipHostMalloc(&block, LANES * DOWNLOAD_CHUNK, hipHostMallocDefault));
        for (int t = 0; t < LANES; ++t) {
            const hipError_t rc = hipStreamCreate(&ctx->download_stream[t]);
            if (rc != hipSuccess) {
                for (int u = 0; u < t; ++u) {
                    (void) hipStreamDestroy(ctx->download_stream[u]);
                    ctx->download_stream[u] = nullptr;
                }
                (void) hipHostFree(block);
                return check_hip(rc, "hipStreamCreate");
            }
        }
        ctx->download_staging = block;
    }
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));  // the source is complete
    const size_t n_chunks = (bytes + DOWNLOAD_CHUNK - 1) / DOWNLOAD_CHUNK;
    hipError_t failed[LANES];
    std::thread lanes[LANES];
    for (int t = 0; t < LANES; ++t) {
        failed[t] = hipSuccess;
        lanes[t] = std::thread([=, &failed] {
            hipError_t rc = hipSetDevice(ctx->device);
            char* staging = (char*) ctx->download_staging + (size_t) t * DOWNLOAD_CHUNK;
            for (size_t c = (size_t) t; rc == hipSuccess && c < n_chunks; c += LANES) {
                const size_t at = c * DOWNLOAD_CHUNK, len = std::min(DOWNLOAD_CHUNK, bytes - at);
                rc = hipMemcpyAsync(staging, d_src + at, len, hipMemcpyDeviceToHost, ctx->download_stream[t]);
                if (rc == hipSuccess) rc = hipStreamSynchronize(ctx->download_stream[t]);
                if (rc == hipSuccess) memcpy(h_dst + at, staging, len);
            }
            failed[t] = rc;
        });
    }
    for (auto& lane : lanes) lane.join();
    for (int t = 0; t < LANES; ++t) SKM_HIP_TRY(failed[t]);
    return SKM_OK;
}
} // namespace

int skm_download(skm_ctx* ctx, void* h_dst, const void* d_src, size_t bytes) {
    SKM_REQUIRE(ctx, "null context");
    if (bytes == 0) return SKM_OK;
    SKM_REQUIRE(h_dst && d_src, "null pointer");
    if (bytes >= DOWNLOAD_LANES_MIN_BYTES) return download_in_lanes(ctx, (char*) h_dst, (const char*) d_src, bytes);
    SKM_HIP_TRY(hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    SKM_HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SKM_OK;
}

int skm_copy(skm_ctx* ctx, void* d_dst, const void* d_src, size_t bytes) {
    SKM_REQUIRE(ctx, "null context");
    if (bytes == 0) return SKM_OK;
    SKM_REQUIRE(d_dst && d_src, "null pointer");
    SKM_HIP_TRY(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return SKM_OK;
}

int skm_fill_u32(skm_ctx* ctx, void* d_dst, uint32_t value, size_t count) {
    SKM_REQUIRE(ctx, "null context");
    if (count == 0) return SKM_OK;
    SKM_REQUIRE(d_dst, "null pointer");
    size_t blocks = (count + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned) blocks), dim3(256), 0, ctx->stream,
                       (uint32_t*) d_dst, value, count);
    return check_hip(hipGetLastError(), "fill_u32_kernel launch");
}

int skm_prof_enable(skm_ctx* ctx, int enabled) {
    SKM_REQUIRE(ctx, "null context");
    if (!enabled) SKM_TRY(resolve_pending(ctx));
    ctx->prof = enabled != 0;
    return SKM_OK;
}

int skm_prof_reset(skm_ctx* ctx) {
    SKM_REQUIRE(ctx, "null context");
    SKM_TRY(resolve_pending(ctx));
    ctx->timers.clear();
    return SKM_OK;
}

int skm_prof_get(skm_ctx* ctx, const char* scope, double* out_ms, uint64_t* out_calls) {
    SKM_REQUIRE(ctx && scope, "null argument");
    SKM_TRY(resolve_pending(ctx));
    auto it = ctx->timers.find(scope);
    if (out_ms) *out_ms = (it == ctx->timers.end()) ? 0.0 : it->second.ms;
    if (out_calls) *out_calls = (it == ctx->timers.end()) ? 0 : it->second.calls;
    return SKM_OK;
}

int skm_prof_dump(skm_ctx* ctx, char* h_buf, size_t buf_len, size_t* out_needed) {
    SKM_REQUIRE(ctx, "null context");
    SKM_TRY(resolve_pending(ctx));
    std::string s;
    char tmp[256];
    for (auto& kv : ctx->timers) {
        snprintf(tmp, sizeof(tmp), "%s=%.6f/%llu;", kv.first.c_str(), kv.second.ms,
                 (unsigned long long) kv.second.calls);
        s += tmp;
    }
    if (out_needed) *out_needed = s.size() + 1;
    if (h_buf && buf_len > 0) {
        size_t ncopy = s.size() < buf_len - 1 ? s.size() : buf_len - 1;
        memcpy(h_buf, s.data(), ncopy);
        h_buf[ncopy] = '\0';
    }
    return SKM_OK;
}

} // extern "C"
