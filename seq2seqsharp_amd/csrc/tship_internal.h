// Internal helpers shared by the translation units of libtship.so: per-thread error string,
// boundary macros that keep C++ exceptions inside the library, the library stream, small device helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_ext.h>

#include <cstdint>
#include <cstdio>
#include <mutex>
#include <stdexcept>
#include <string>

#include "../../include/tship.h"

namespace tship {

void set_last_error(const std::string& msg);

struct Error : std::runtime_error {
    explicit Error(const std::string& m) : std::runtime_error(m) {}
};

#define TSHIP_CHECK_HIP(expr)                                                                         \
    do {                                                                                              \
        hipError_t _e = (expr);                                                                       \
        if (_e != hipSuccess)                                                                         \
            throw ::tship::Error(std::string(#expr) + " failed: " + hipGetErrorString(_e));           \
    } while (0)

#define TSHIP_REQUIRE(cond, msg)                                                                      \
    do {                                                                                              \
        if (!(cond)) throw ::tship::Error(std::string(msg));                                          \
    } while (0)

// One lock for every exported call that touches the device: the library drives one ordered stream, and a call may span
// many launches that must not interleave with another thread's (a HIP graph capture records whatever lands on the stream
// meanwhile; a model's buffers are written by consecutive kernels).  Callers on several threads, as the reference's
// Parallel.For over devices (BaseSeq2SeqFramework.cs:912-941), are serialised here; the lock is recursive because
// exported calls nest.
std::recursive_mutex& api_mutex();

// Every exported function is wrapped: 1 on success, 0 on failure with the message stored per thread.
#define TSHIP_BEGIN try { std::lock_guard<std::recursive_mutex> tship_api_lock(::tship::api_mutex());
#define TSHIP_END                                                                                     \
    return 1;                                                                                         \
    }                                                                                                 \
    catch (const std::exception& e) {                                                                 \
        ::tship::set_last_error(e.what());                                                            \
        return 0;                                                                                     \
    }                                                                                                 \
    catch (...) {                                                                                     \
        ::tship::set_last_error("unknown native exception");                                          \
        return 0;                                                                                     \
    }

// The library's ordered stream (created by TSHip_Init, default priority).
hipStream_t stream();
void ensure_init();
int current_device();          // device the library was initialised on, -1 before TSHip_Init
void noalloc_device_setup(int device);   // tship_ops.hip: address of the fixed scratch array, once per device
int n_compute_units();
// device memory for the library's own use: blocks of the size-class pool behind TSHip_Malloc / TSHip_Free (no driver call
// when a cached block fits), and a plain allocation that, on failure, releases what the pool only caches and tries again
void* pool_alloc(size_t bytes);
void pool_release(void* p);
void* device_malloc_retry(size_t bytes);

typedef _Float16 half_t;
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "libtship's device code is written for gfx950 only: MFMA shapes, direct-to-LDS loads, and cross-block exchanges whose ordering rests on this target's instruction behaviour"
#endif
typedef half_t half8 __attribute__((ext_vector_type(8)));
typedef half_t half4 __attribute__((ext_vector_type(4)));
typedef half_t half2v __attribute__((ext_vector_type(2)));
typedef half_t half4v __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

__host__ __device__ static inline long round_up(long v, long m) { return (v + m - 1) / m * m; }
__host__ __device__ static inline long ceil_div(long a, long b) { return (a + b - 1) / b; }

// ------------------------------------------------------------------------------------------------
// reductions
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// 256-thread block sum; s is LDS scratch of 4 floats; every thread gets the result
// A load of data that the launch reads exactly once (weight fragments of the decode GEMMs, cached keys and values of the
// decode attention): requested as non-temporal, so that the caches on the way do not keep a copy at the cost of lines that
// are read again (activation fragments, partial sums).  Measured at batch 32 x 1100 cached positions: the attention
// launch 15.8 -> 14.1 us, the vocabulary projection 27.5 -> 25.4 us, the decode step 0.843 -> 0.813 ms.
template <typename T>
__device__ __forceinline__ T load_once(const T* p) { return __builtin_nontemporal_load(p); }

__device__ __forceinline__ float block_sum_256(float v, float* s) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = v;
    __syncthreads();
    return (s[0] + s[1]) + (s[2] + s[3]);
}


}  // namespace tship
