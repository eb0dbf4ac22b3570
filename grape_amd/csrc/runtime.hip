// Runtime part of the C ABI: device selection, error text, memory helpers, the scratch pool and
// the two roofline micro-benchmarks (stream copy, v_mad_u64_u32 issue rate).
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <map>
#include <mutex>
#include <thread>
#include <vector>
#include "common.hpp"

namespace grape {

static thread_local char g_err[512] = "";
static bool g_init = false;

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}
bool initialised() { return g_init; }

static bool g_prof = false;
static hipEvent_t g_prof_ev[8];
static int g_prof_n = 0, g_prof_cap = 0;
bool profiling() { return g_prof; }
void profile_begin() { g_prof_n = 0; }
int profile_mark(hipStream_t s) {
    if (!g_prof || g_prof_n >= 8) return GRAPE_OK;
    if (g_prof_n >= g_prof_cap) {
        GRAPE_HIP_CHECK(hipEventCreate(&g_prof_ev[g_prof_cap]));
        g_prof_cap++;
    }
    GRAPE_HIP_CHECK(hipEventRecord(g_prof_ev[g_prof_n], s));
    g_prof_n++;
    return GRAPE_OK;
}

__global__ void __launch_bounds__(kBlock) zero_words_kernel(uint32_t* p, size_t words) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < words; i += (size_t)gridDim.x * kBlock) p[i] = 0;
}

__global__ void __launch_bounds__(kBlock) zero_bytes_kernel(uint8_t* p, size_t bytes) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < bytes; i += (size_t)gridDim.x * kBlock) p[i] = 0;
}

int zero_fill(void* d_ptr, size_t bytes, hipStream_t s) {
    if (bytes == 0) return GRAPE_OK;
    if ((bytes & 3) == 0 && (reinterpret_cast<uintptr_t>(d_ptr) & 3) == 0) {
        const size_t words = bytes / 4;
        const size_t want = (words + kBlock - 1) / kBlock;
        zero_words_kernel<<<(unsigned)(want < 4096 ? want : 4096), kBlock, 0, s>>>((uint32_t*)d_ptr, words);
        GRAPE_LAUNCH_CHECK();
        return GRAPE_OK;
    }
    // sizes or addresses that are no multiple of 4 (no caller inside this library): byte by byte
    const size_t want = (bytes + kBlock - 1) / kBlock;
    zero_bytes_kernel<<<(unsigned)(want < 4096 ? want : 4096), kBlock, 0, s>>>((uint8_t*)d_ptr, bytes);
    GRAPE_LAUNCH_CHECK();
    return GRAPE_OK;
}

size_t alloc_cache_release();   // gives the blocks kept by grape_free back to the driver
int noalloc_setup();            // proto_kernels.hip: looks up the static scratch array of the current device

// One pool per stream: a buffer is only ever used by kernels of the stream it was handed out for,
// so calls on different streams (from one host thread or from several) never share scratch
// memory, and growing a buffer only has to wait for its own stream.  The bookkeeping is behind a
// mutex; one host thread per stream stays the rule (two threads that interleave calls on the SAME
// stream would still share its buffers).
struct StreamPool {
    void* ptr[kNumSlots] = {nullptr};
    size_t bytes[kNumSlots] = {0};
};
static std::mutex g_scratch_mu;
static std::map<hipStream_t, StreamPool>* g_pools = nullptr;

int scratch_get(ScratchSlot slot, size_t bytes, void** out, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_pools) g_pools = new std::map<hipStream_t, StreamPool>();
    StreamPool& pool = (*g_pools)[stream];
    if (bytes > pool.bytes[slot]) {
        if (pool.ptr[slot]) {
            GRAPE_HIP_CHECK(hipStreamSynchronize(stream));
            GRAPE_HIP_CHECK(hipFree(pool.ptr[slot]));
            pool.ptr[slot] = nullptr;
            pool.bytes[slot] = 0;
        }
        size_t want = bytes < (1u << 20) ? (1u << 20) : bytes;
        hipError_t e = hipMalloc(&pool.ptr[slot], want);
        if (e != hipSuccess && alloc_cache_release() > 0) {
            (void)hipGetLastError();
            e = hipMalloc(&pool.ptr[slot], want);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();
            pool.ptr[slot] = nullptr;
            set_error("scratch allocation of %zu bytes failed: %s", want, hipGetErrorString(e));
            return GRAPE_ENOMEM;
        }
        pool.bytes[slot] = want;
    }
    *out = pool.ptr[slot];
    return GRAPE_OK;
}


// 16-byte-per-lane streaming copy, grid-stride
__global__ void __launch_bounds__(256) copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

// 8 independent multiply-add chains per lane keep the multiplier pipe full; each chain feeds
// its own low word back as the multiplicand so nothing can be hoisted or shared.
__global__ void __launch_bounds__(256) mad_kernel(uint64_t* out, int inner, uint32_t seed) {
    uint32_t a = threadIdx.x * 2654435761u + seed, b = (blockIdx.x * 40503u + 12345u + seed) | 1u;
    uint64_t c[8];
#pragma unroll
    for (int k = 0; k < 8; k++) c[k] = (uint64_t)(a + k) * 0x9e3779b97f4a7c15ull;
    for (int it = 0; it < inner; it++) {
#pragma unroll
        for (int rep = 0; rep < 8; rep++) {
#pragma unroll
            for (int k = 0; k < 8; k++) c[k] = (uint64_t)(uint32_t)c[k] * b + c[k];
        }
    }
    uint64_t r = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) r ^= c[k];
    if (r == 0x123456789abcdefull) out[0] = r;   // practically never; keeps the chains alive
}

// Block cache of grape_malloc / grape_free.  The host classes allocate and free a tensor per
// call as the reference does (cudaMalloc / cudaFree, src/fr-tensor.cu:371-374, :235-241); hipMalloc
// and hipFree take tens of microseconds for small blocks and from a millisecond to hundreds of them
// for multi-GiB ones, so a freed block is kept (up to a total that GRAPE_ALLOC_CACHE_GIB sets,
// 32 GiB by default, 0 = off) and handed out again to a request of exactly its size.  hipFree waits for the device; a caller
// may rely on that and free a buffer that queued kernels still use, so the wait happens when a
// cached block is handed out again instead.
static std::mutex g_alloc_mu;
// A kept block may only be handed out again once the work that was queued when it was freed has
// finished - what hipFree would have waited for.  Waiting for the whole device at that point
// (hipDeviceSynchronize) would also wait for work queued LATER on other streams, e.g. for the rounds
// a lookup has queued on its side streams while its commitments allocate on the default stream; so
// the free records an event on every stream the library knows (the default stream and the streams
// of grape_stream_create) and the reuse waits for those events only.  Once a caller has brought a
// stream of its own the cache cannot know what that stream still runs and goes back to waiting for
// the device.
constexpr int kMaxLibStreams = 16;
struct CachedBlock {
    void* p = nullptr;
    hipEvent_t ev[1 + kMaxLibStreams];
    int nev = 0;
    bool whole_device = false;
};
static std::map<void*, size_t>* g_live = nullptr;                    // blocks handed out by grape_malloc
static std::multimap<size_t, CachedBlock>* g_cached = nullptr;       // freed blocks kept for reuse
static size_t g_cached_bytes = 0;
static std::vector<hipEvent_t>* g_event_pool = nullptr;
static hipStream_t g_lib_streams[kMaxLibStreams];
static std::atomic<int> g_n_lib_streams{0};
static std::atomic<bool> g_foreign_stream{false};
// Blocks are also freed while the process exits (destructors of static objects that own tensors).
// By then layers under this one may be half torn down - a profiler's per-thread stream bookkeeping
// is gone once the main thread's thread-local objects have been destroyed, and a stream call then
// aborts - so from that point on a free records nothing.  The point is marked by the destructor of a
// thread-local object of the thread that initialised the library: thread-local objects of the
// exiting thread are destroyed before any static object.
static std::atomic<bool> g_exit_started{false};
static std::atomic<bool> g_first_thread_set{false};
static std::thread::id g_first_thread;
struct ExitSentinel {
    ~ExitSentinel() {
        if (g_first_thread_set.load() && std::this_thread::get_id() == g_first_thread) g_exit_started.store(true);
    }
};
static void touch_exit_sentinel() {
    thread_local ExitSentinel sentinel;
    (void)&sentinel;
    if (!g_first_thread_set.load()) {
        g_first_thread = std::this_thread::get_id();
        g_first_thread_set.store(true);
    }
}
static size_t alloc_cache_cap() {
    static size_t cap = [] {
        size_t gib = 32;
        if (const char* e = getenv("GRAPE_ALLOC_CACHE_GIB")) {
            char* end = nullptr;
            unsigned long long v = strtoull(e, &end, 10);
            if (end != e) gib = (size_t)v;
        }
        return gib << 30;
    }();
    return cap;
}
static void alloc_tables() {
    if (!g_live) {
        g_live = new std::map<void*, size_t>();
        g_cached = new std::multimap<size_t, CachedBlock>();
        g_event_pool = new std::vector<hipEvent_t>();
    }
}
static bool take_event(hipEvent_t* out) {
    if (!g_event_pool->empty()) {
        *out = g_event_pool->back();
        g_event_pool->pop_back();
        return true;
    }
    if (hipEventCreateWithFlags(out, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return true;
}
// marks the point up to which the block may still be in use: an event on every known stream
static void stamp_block(CachedBlock& b) {
    b.nev = 0;
    const int n = g_n_lib_streams.load();
    // with the default stream alone there is nothing a wait for the device would wait for needlessly,
    // and it costs less than an event per free
    b.whole_device = n == 0 || g_foreign_stream.load() || g_exit_started.load();
    if (b.whole_device) return;
    for (int i = -1; i < n; i++) {
        hipEvent_t e;
        if (!take_event(&e) || hipEventRecord(e, i < 0 ? (hipStream_t) nullptr : g_lib_streams[i]) != hipSuccess) {
            (void)hipGetLastError();
            b.whole_device = true;
            break;
        }
        b.ev[b.nev++] = e;
    }
}
static int wait_block(CachedBlock& b) {
    if (b.whole_device) GRAPE_HIP_CHECK(hipDeviceSynchronize());
    for (int i = 0; i < b.nev; i++) {
        if (!b.whole_device) GRAPE_HIP_CHECK(hipEventSynchronize(b.ev[i]));
        g_event_pool->push_back(b.ev[i]);
    }
    b.nev = 0;
    return GRAPE_OK;
}
// gives every cached block back to the driver; returns the bytes released
static size_t alloc_cache_release_locked() {
    size_t n = g_cached_bytes;
    if (g_cached) {
        for (auto& e : *g_cached) {
            (void)hipFree(e.second.p);                    // waits for the device
            for (int i = 0; i < e.second.nev; i++) g_event_pool->push_back(e.second.ev[i]);
        }
        g_cached->clear();
    }
    g_cached_bytes = 0;
    return n;
}

void note_stream(hipStream_t s) {
    if (g_foreign_stream.load(std::memory_order_relaxed)) return;
    const int n = g_n_lib_streams.load(std::memory_order_acquire);
    for (int i = 0; i < n; i++)
        if (g_lib_streams[i] == s) return;
    g_foreign_stream.store(true);
}

size_t alloc_cache_release() {
    std::lock_guard<std::mutex> lock(g_alloc_mu);
    return alloc_cache_release_locked();
}

}  // namespace grape

using namespace grape;

extern "C" {

int grape_init(int device) {
    GRAPE_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    GRAPE_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("grape_init: device %d is %s, this library is built for gfx950 only", device, prop.gcnArchName);
        return GRAPE_EINVAL;
    }
    g_init = true;
    touch_exit_sentinel();
    return noalloc_setup();
}
const char* grape_last_error(void) { return g_err; }
int grape_stream_sync(grape_stream_t s) {
    GRAPE_HIP_CHECK(hipStreamSynchronize(as_stream(s)));
    return GRAPE_OK;
}
int grape_malloc(void** p, size_t bytes) {
    GRAPE_REQUIRE(p != nullptr, "null output pointer");
    if (bytes == 0) bytes = 1;
    std::lock_guard<std::mutex> lock(g_alloc_mu);
    alloc_tables();
    auto it = g_cached->find(bytes);
    if (it != g_cached->end()) {
        CachedBlock b = it->second;
        g_cached->erase(it);
        g_cached_bytes -= bytes;
        int rc = wait_block(b);                           // what hipFree would have waited for
        (*g_live)[b.p] = bytes;
        *p = b.p;
        return rc;
    }
    hipError_t e = hipMalloc(p, bytes);
    if (e != hipSuccess && alloc_cache_release_locked() > 0) {
        (void)hipGetLastError();
        e = hipMalloc(p, bytes);                          // once more with the cache given back
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        return GRAPE_ENOMEM;
    }
    (*g_live)[*p] = bytes;
    return GRAPE_OK;
}
int grape_free(void* p) {
    if (!p) return GRAPE_OK;
    std::lock_guard<std::mutex> lock(g_alloc_mu);
    touch_exit_sentinel();
    alloc_tables();
    auto it = g_live->find(p);
    if (it != g_live->end()) {
        const size_t bytes = it->second;
        g_live->erase(it);
        if (g_cached_bytes + bytes <= alloc_cache_cap()) {
            CachedBlock b;
            b.p = p;
            stamp_block(b);
            g_cached->emplace(bytes, b);
            g_cached_bytes += bytes;
            return GRAPE_OK;
        }
    }
    GRAPE_HIP_CHECK(hipFree(p));
    return GRAPE_OK;
}
int grape_alloc_cache_release(size_t* bytes_released) {
    std::lock_guard<std::mutex> lock(g_alloc_mu);
    alloc_tables();
    GRAPE_HIP_CHECK(hipDeviceSynchronize());
    const size_t n = alloc_cache_release_locked();
    if (bytes_released) *bytes_released = n;
    return GRAPE_OK;
}
// A payload of at most 1 KiB travels as the argument of a kernel that writes it: queued on the
// stream like any other work, nothing to wait for, and the host buffer is free at once (the
// launch has copied the argument).  A copy from pageable host memory would make the host wait for
// everything the stream still holds - once per scalar handed to a kernel.
struct SmallPayload { uint32_t w[256]; };
__global__ void __launch_bounds__(256) poke_kernel(uint32_t* dst, SmallPayload p, uint32_t words) {
    if (threadIdx.x < words) dst[threadIdx.x] = p.w[threadIdx.x];
}
int grape_memcpy_h2d(void* d, const void* s, size_t bytes, grape_stream_t st) {
    if (!bytes) return GRAPE_OK;
    if (bytes <= sizeof(SmallPayload) && (bytes & 3) == 0 && (reinterpret_cast<uintptr_t>(d) & 3) == 0) {
        GRAPE_REQUIRE(d != nullptr && s != nullptr, "null pointer");
        SmallPayload p;
        memcpy(p.w, s, bytes);
        poke_kernel<<<1, 256, 0, as_stream(st)>>>((uint32_t*)d, p, (uint32_t)(bytes / 4));
        GRAPE_LAUNCH_CHECK();
        return GRAPE_OK;
    }
    GRAPE_HIP_CHECK(hipMemcpyAsync(d, s, bytes, hipMemcpyHostToDevice, as_stream(st)));
    GRAPE_HIP_CHECK(hipStreamSynchronize(as_stream(st)));   // the host buffer may be reused at once
    return GRAPE_OK;
}
int grape_memcpy_d2h(void* d, const void* s, size_t bytes, grape_stream_t st) {
    if (!bytes) return GRAPE_OK;
    GRAPE_HIP_CHECK(hipMemcpyAsync(d, s, bytes, hipMemcpyDeviceToHost, as_stream(st)));
    GRAPE_HIP_CHECK(hipStreamSynchronize(as_stream(st)));
    return GRAPE_OK;
}
int grape_memcpy_d2d(void* d, const void* s, size_t bytes, grape_stream_t st) {
    if (!bytes) return GRAPE_OK;
    GRAPE_HIP_CHECK(hipMemcpyAsync(d, s, bytes, hipMemcpyDeviceToDevice, as_stream(st)));
    return GRAPE_OK;
}
int grape_memset_zero(void* d, size_t bytes, grape_stream_t st) {
    if (!bytes) return GRAPE_OK;
    return zero_fill(d, bytes, as_stream(st));
}

int grape_profile_enable(int on) {
    g_prof = on != 0;
    g_prof_n = 0;
    return GRAPE_OK;
}
int grape_profile_last(float* ms, int cap, int* n) {
    GRAPE_REQUIRE(ms != nullptr && n != nullptr, "null output");
    *n = 0;
    for (int i = 0; i + 1 < g_prof_n && i < cap; i++) {
        GRAPE_HIP_CHECK(hipEventSynchronize(g_prof_ev[i + 1]));
        GRAPE_HIP_CHECK(hipEventElapsedTime(&ms[i], g_prof_ev[i], g_prof_ev[i + 1]));
        *n = i + 1;
    }
    return GRAPE_OK;
}

// A stream of the default priority that does not synchronise with the legacy default stream; its
// scratch pool is dropped with it.
int grape_stream_create(grape_stream_t* out) {
    GRAPE_REQUIRE(out != nullptr, "null output");
    hipStream_t s;
    std::lock_guard<std::mutex> lock(g_alloc_mu);
    const int n = g_n_lib_streams.load();
    GRAPE_REQUIRE(n < kMaxLibStreams, "too many streams");
    GRAPE_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    g_lib_streams[n] = s;
    g_n_lib_streams.store(n + 1, std::memory_order_release);
    *out = reinterpret_cast<grape_stream_t>(s);
    return GRAPE_OK;
}
int grape_stream_destroy(grape_stream_t st) {
    hipStream_t s = as_stream(st);
    GRAPE_REQUIRE(s != nullptr, "the default stream cannot be destroyed");
    GRAPE_HIP_CHECK(hipStreamSynchronize(s));
    {
        std::lock_guard<std::mutex> lock(g_scratch_mu);
        if (g_pools) {
            auto it = g_pools->find(s);
            if (it != g_pools->end()) {
                for (int k = 0; k < kNumSlots; k++)
                    if (it->second.ptr[k]) (void)hipFree(it->second.ptr[k]);
                g_pools->erase(it);
            }
        }
    }
    {
        // the blocks freed while this stream existed carry events recorded on it: wait for the device
        // once, so that those events count as reached, and forget the stream
        std::lock_guard<std::mutex> lock(g_alloc_mu);
        GRAPE_HIP_CHECK(hipDeviceSynchronize());
        const int n = g_n_lib_streams.load();
        for (int i = 0; i < n; i++) {
            if (g_lib_streams[i] == s) {
                g_lib_streams[i] = g_lib_streams[n - 1];
                g_n_lib_streams.store(n - 1, std::memory_order_release);
                break;
            }
        }
    }
    GRAPE_HIP_CHECK(hipStreamDestroy(s));
    return GRAPE_OK;
}
int grape_stream_wait_event(grape_stream_t st, void* ev) {
    GRAPE_REQUIRE(ev != nullptr, "null event");
    GRAPE_HIP_CHECK(hipStreamWaitEvent(as_stream(st), (hipEvent_t)ev, 0));
    return GRAPE_OK;
}

int grape_event_create(void** ev) {
    hipEvent_t e;
    GRAPE_HIP_CHECK(hipEventCreate(&e));
    *ev = e;
    return GRAPE_OK;
}
int grape_event_destroy(void* ev) {
    GRAPE_HIP_CHECK(hipEventDestroy((hipEvent_t)ev));
    return GRAPE_OK;
}
int grape_event_record(void* ev, grape_stream_t s) {
    GRAPE_HIP_CHECK(hipEventRecord((hipEvent_t)ev, as_stream(s)));
    return GRAPE_OK;
}
int grape_event_elapsed_ms(float* ms, void* a, void* b) {
    GRAPE_HIP_CHECK(hipEventSynchronize((hipEvent_t)b));
    GRAPE_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)a, (hipEvent_t)b));
    return GRAPE_OK;
}

int grape_bench_copy(void* d_dst, const void* d_src, size_t bytes, int iters, float* ms, grape_stream_t st) {
    GRAPE_REQUIRE(d_dst && d_src && ms && iters > 0 && bytes % 16 == 0, "bad arguments");
    hipEvent_t e0, e1;
    GRAPE_HIP_CHECK(hipEventCreate(&e0));
    GRAPE_HIP_CHECK(hipEventCreate(&e1));
    size_t n16 = bytes / 16;
    unsigned grid = kNumCU * 16;
    copy_kernel<<<grid, 256, 0, as_stream(st)>>>((uint4*)d_dst, (const uint4*)d_src, n16);   // warm-up
    GRAPE_HIP_CHECK(hipEventRecord(e0, as_stream(st)));
    for (int i = 0; i < iters; i++) copy_kernel<<<grid, 256, 0, as_stream(st)>>>((uint4*)d_dst, (const uint4*)d_src, n16);
    GRAPE_HIP_CHECK(hipEventRecord(e1, as_stream(st)));
    GRAPE_HIP_CHECK(hipEventSynchronize(e1));
    GRAPE_LAUNCH_CHECK();
    float t;
    GRAPE_HIP_CHECK(hipEventElapsedTime(&t, e0, e1));
    *ms = t / iters;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return GRAPE_OK;
}

int grape_bench_mad_u64_u32(int blocks, int inner, int iters, double* mads_per_s, grape_stream_t st) {
    GRAPE_REQUIRE(blocks > 0 && inner > 0 && iters > 0 && mads_per_s, "bad arguments");
    void* out;
    int rc = scratch_get(kSlotMisc, 64, &out, as_stream(st));
    if (rc) return rc;
    hipEvent_t e0, e1;
    GRAPE_HIP_CHECK(hipEventCreate(&e0));
    GRAPE_HIP_CHECK(hipEventCreate(&e1));
    mad_kernel<<<blocks, 256, 0, as_stream(st)>>>((uint64_t*)out, inner, 1u);
    GRAPE_HIP_CHECK(hipEventRecord(e0, as_stream(st)));
    for (int i = 0; i < iters; i++) mad_kernel<<<blocks, 256, 0, as_stream(st)>>>((uint64_t*)out, inner, (uint32_t)i);
    GRAPE_HIP_CHECK(hipEventRecord(e1, as_stream(st)));
    GRAPE_HIP_CHECK(hipEventSynchronize(e1));
    GRAPE_LAUNCH_CHECK();
    float t;
    GRAPE_HIP_CHECK(hipEventElapsedTime(&t, e0, e1));
    double mads = (double)blocks * 256.0 * (double)inner * 64.0 * (double)iters;
    *mads_per_s = mads / (t * 1e-3);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return GRAPE_OK;
}

}  // extern "C"
