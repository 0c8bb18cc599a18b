// Runtime half of the C ABI: initialisation, device memory and synchronous host<->device copies.
// Mirrors what a managed HipAllocator / HipStorage needs (TensorSharp/IAllocator.cs:13-20,
// TensorSharp/Storage.cs:32-47); the error convention follows TensorSharp.GGML.Native/ggml_ops.cpp:211-224.
#include "tship_internal.h"

#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace tship {

static thread_local std::string t_last_error;
void set_last_error(const std::string& msg) { t_last_error = msg; }

static std::recursive_mutex g_api_mutex;
std::recursive_mutex& api_mutex() { return g_api_mutex; }

static std::mutex g_init_mutex;
static bool g_initialised = false;
static int g_device = -1;
static hipStream_t g_stream = nullptr;
static int g_cus = 0;

hipStream_t stream() { return g_stream; }
int current_device() { return g_initialised ? g_device : -1; }
int n_compute_units() { return g_cus; }

static void init_locked(int device_id) {
    if (g_initialised) {
        if (device_id != g_device)
            throw Error("TSHip_Init: already initialised on device " + std::to_string(g_device) +
                        "; a process drives one device");
        return;
    }
    int count = 0;
    TSHIP_CHECK_HIP(hipGetDeviceCount(&count));
    if (count <= 0) throw Error("TSHip_Init: no HIP device is visible");
    if (device_id < 0 || device_id >= count) throw Error("TSHip_Init: device id out of range");
    TSHIP_CHECK_HIP(hipSetDevice(device_id));
    hipDeviceProp_t prop;
    TSHIP_CHECK_HIP(hipGetDeviceProperties(&prop, device_id));
    std::string arch = prop.gcnArchName;
    if (arch.rfind("gfx950", 0) != 0)
        throw Error("TSHip_Init: this library is built for gfx950 (MI355X); device reports " + arch);
    g_cus = prop.multiProcessorCount;
    noalloc_device_setup(device_id);
    TSHIP_CHECK_HIP(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    g_device = device_id;
    g_initialised = true;
}

void ensure_init() {
    std::lock_guard<std::mutex> lk(g_init_mutex);
    if (!g_initialised) init_locked(0);
}

// ------------------------------------------------------------------------------------------------
// Device memory pool behind TSHip_Malloc / TSHip_Free (the role of TensorSharp.CUDA/ContextState/PoolingDeviceAllocator.cs:
// tensors come and go about 45 times per layer and step on the per-op surface, and hipMalloc / hipFree cost tens of
// microseconds each and synchronise the device).
// Blocks are cached by size class and never returned to the driver while the process runs (TSHip_PoolTrim and an
// allocation failure release them).  A freed block may be handed out again at once without waiting for the GPU: every
// kernel and copy of this library runs on the one library stream, so whatever still reads the block was enqueued before
// whatever the next owner enqueues.
// Size classes: multiples of 256 bytes up to 4 KiB, then four classes per power of two (a request just above a power of two rounds up by a quarter: at most 25 % slack).
// ------------------------------------------------------------------------------------------------
static std::mutex g_pool_mutex;
static std::unordered_map<void*, size_t> g_pool_live;                 // block -> class size
static std::map<size_t, std::vector<void*>> g_pool_free;              // class size -> cached blocks
static size_t g_pool_device_allocs = 0, g_pool_bytes_cached = 0, g_pool_bytes_live = 0;

static size_t pool_class(size_t bytes) {
    if (bytes <= 4096) return (bytes + 255) / 256 * 256;
    size_t p = 4096;
    while (p * 2 < bytes) p *= 2;                                        // p < bytes <= 2p
    const size_t step = p / 4;
    return p + (bytes - p + step - 1) / step * step;
}

static void pool_release_cached_locked() {
    for (auto& kv : g_pool_free) for (void* p : kv.second) (void)hipFree(p);
    g_pool_free.clear();
    g_pool_bytes_cached = 0;
}

static void* pool_malloc(size_t bytes) {
    const size_t cls = pool_class(bytes == 0 ? 4 : bytes);
    std::lock_guard<std::mutex> lk(g_pool_mutex);
    auto it = g_pool_free.find(cls);
    if (it != g_pool_free.end() && !it->second.empty()) {
        void* p = it->second.back(); it->second.pop_back();
        g_pool_bytes_cached -= cls; g_pool_bytes_live += cls;
        g_pool_live[p] = cls;
        return p;
    }
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, cls);
    if (e != hipSuccess) {
        // give the cached blocks back and try once more (the GPU may still be using them: wait for it first)
        (void)hipGetLastError();
        (void)hipStreamSynchronize(stream());
        pool_release_cached_locked();
        e = hipMalloc(&p, cls);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        throw Error("out of device memory: hipMalloc(" + std::to_string(cls) + " bytes) failed: " + hipGetErrorString(e));
    }
    ++g_pool_device_allocs;
    g_pool_bytes_live += cls;
    g_pool_live[p] = cls;
    return p;
}

static void pool_free(void* p) {
    std::lock_guard<std::mutex> lk(g_pool_mutex);
    auto it = g_pool_live.find(p);
    if (it == g_pool_live.end()) throw Error("TSHip_Free: pointer was not allocated by TSHip_Malloc (or was freed before)");
    const size_t cls = it->second;
    g_pool_live.erase(it);
    g_pool_free[cls].push_back(p);
    g_pool_bytes_live -= cls; g_pool_bytes_cached += cls;
}

// for the library's own temporaries and long-lived buffers (declared in tship_internal.h)
void* pool_alloc(size_t bytes) { return pool_malloc(bytes); }
void pool_release(void* p) { pool_free(p); }
void* device_malloc_retry(size_t bytes) {
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
        // memory that is only cached by the pool is not lost: wait for the GPU, give the cached blocks back, try once more
        (void)hipGetLastError();
        (void)hipStreamSynchronize(stream());
        { std::lock_guard<std::mutex> lk(g_pool_mutex); pool_release_cached_locked(); }
        e = hipMalloc(&p, bytes);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        throw Error("out of device memory: hipMalloc(" + std::to_string(bytes) + " bytes) failed: " + hipGetErrorString(e));
    }
    return p;
}

}  // namespace tship

using namespace tship;

extern "C" {

TSHIP_API const char* TSHip_GetLastError(void) { return t_last_error.c_str(); }

TSHIP_API int TSHip_GetDeviceCount(int* count) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(count != nullptr, "TSHip_GetDeviceCount: count is null");
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e != hipSuccess) { c = 0; (void)hipGetLastError(); }
    *count = c;
    TSHIP_END
}

TSHIP_API int TSHip_Init(int device_id) {
    TSHIP_BEGIN
    std::lock_guard<std::mutex> lk(g_init_mutex);
    init_locked(device_id);
    TSHIP_END
}

TSHIP_API int TSHip_Malloc(void** ptr, size_t bytes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(ptr != nullptr, "TSHip_Malloc: ptr is null");
    ensure_init();
    *ptr = nullptr;
    *ptr = pool_malloc(bytes);
    TSHIP_END
}

TSHIP_API int TSHip_Free(void* ptr) {
    TSHIP_BEGIN
    if (ptr) {
        ensure_init();
        pool_free(ptr);
    }
    TSHIP_END
}

TSHIP_API int TSHip_PoolTrim(void) {
    TSHIP_BEGIN
    ensure_init();
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    std::lock_guard<std::mutex> lk(g_pool_mutex);
    pool_release_cached_locked();
    TSHIP_END
}

TSHIP_API int TSHip_GetPoolStats(size_t* device_allocations, size_t* bytes_in_use, size_t* bytes_cached) {
    TSHIP_BEGIN
    std::lock_guard<std::mutex> lk(g_pool_mutex);
    if (device_allocations) *device_allocations = g_pool_device_allocs;
    if (bytes_in_use) *bytes_in_use = g_pool_bytes_live;
    if (bytes_cached) *bytes_cached = g_pool_bytes_cached;
    TSHIP_END
}

TSHIP_API int TSHip_MemcpyH2D(void* dst, const void* src, size_t bytes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(dst && src, "TSHip_MemcpyH2D: null pointer");
    ensure_init();
    TSHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_END
}

TSHIP_API int TSHip_MemcpyD2H(void* dst, const void* src, size_t bytes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(dst && src, "TSHip_MemcpyD2H: null pointer");
    ensure_init();
    TSHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, stream()));
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_END
}

TSHIP_API int TSHip_MemcpyD2D(void* dst, const void* src, size_t bytes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(dst && src, "TSHip_MemcpyD2D: null pointer");
    ensure_init();
    TSHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream()));
    TSHIP_END
}

TSHIP_API int TSHip_Memset(void* dst, int value, size_t bytes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(dst != nullptr, "TSHip_Memset: null pointer");
    ensure_init();
    TSHIP_CHECK_HIP(hipMemsetAsync(dst, value, bytes, stream()));
    TSHIP_END
}

TSHIP_API int TSHip_Synchronize(void) {
    TSHIP_BEGIN
    ensure_init();
    TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
    TSHIP_END
}

TSHIP_API int TSHip_GetMemInfo(size_t* free_bytes, size_t* total_bytes) {
    TSHIP_BEGIN
    TSHIP_REQUIRE(free_bytes && total_bytes, "TSHip_GetMemInfo: null pointer");
    ensure_init();
    TSHIP_CHECK_HIP(hipMemGetInfo(free_bytes, total_bytes));
    TSHIP_END
}

}  // extern "C"
