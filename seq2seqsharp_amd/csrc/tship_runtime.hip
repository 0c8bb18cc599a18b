// Runtime half of the C ABI: initialisation, device memory and synchronous host<->device copies.
// Mirrors what a managed HipAllocator / HipStorage needs (TensorSharp/IAllocator.cs:13-20,
// TensorSharp/Storage.cs:32-47); the error convention follows TensorSharp.GGML.Native/ggml_ops.cpp:211-224.
#include "tship_internal.h"

#include <mutex>

namespace tship {

static thread_local std::string t_last_error;
void set_last_error(const std::string& msg) { t_last_error = msg; }

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
    if (bytes == 0) bytes = 4;
    hipError_t e = hipMalloc(ptr, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        throw Error("out of device memory: hipMalloc(" + std::to_string(bytes) + " bytes) failed: " + hipGetErrorString(e));
    }
    TSHIP_END
}

TSHIP_API int TSHip_Free(void* ptr) {
    TSHIP_BEGIN
    if (ptr) {
        ensure_init();
        TSHIP_CHECK_HIP(hipStreamSynchronize(stream()));
        TSHIP_CHECK_HIP(hipFree(ptr));
    }
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
