// Shared declarations of the gfx950 kernel library.
//
// Every entry point is `extern "C"`, takes raw device pointers, sizes and a
// HIP stream, checks on the host that the sizes fit what its kernel and grid
// assume, and returns 0 or a non-zero code after storing a message that
// `somi_last_error()` returns.  No entry point allocates device memory.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16;

enum SomiDtype { SOMI_F32 = 0, SOMI_BF16 = 1 };

extern "C" const char* somi_last_error();
int somi_fail(const char* fmt, ...);   // stores the message, returns 1

#define SOMI_REQUIRE(cond, ...)                    \
    do {                                           \
        if (!(cond)) return somi_fail(__VA_ARGS__); \
    } while (0)

#define SOMI_LAUNCH_CHECK(name)                                                         \
    do {                                                                                \
        hipError_t err__ = hipGetLastError();                                           \
        if (err__ != hipSuccess)                                                        \
            return somi_fail("%s: launch failed: %s", name, hipGetErrorString(err__)); \
    } while (0)

// Element access as float, whatever the storage type.
__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) { return (bf16)v; }

// Cache policy bits of a buffer load (its last argument) for data that is read once, such as a weight matrix
// streamed through a product of a few rows: "non-temporal" tells the caches not to keep the lines.  A streaming read
// of 2 GiB measures 6.6 TB/s with it and 5.9 without on an MI355X.
#define SOMI_LOAD_ONCE 2

// Compute units of the current device, asked once per device (256 if the device cannot be asked): what the launch
// shapes size their workgroup counts by.
int somi_units();

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Sum / max over a workgroup of NT threads (NT a multiple of 64, at most
// 1024) through wave shuffles and one LDS array of 16 floats.  The order of
// the additions depends on NT only, so a row's result does not depend on what
// else is in the launch.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
template <int NT> __device__ __forceinline__ float block_sum(float v, float* red /*[16]*/) {
    v = wave_sum(v);
    if (NT == 64) return v;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < NT / 64; ++i) total += red[i];
    return total;
}
template <int NT> __device__ __forceinline__ float block_max(float v, float* red /*[16]*/) {
    v = wave_max(v);
    if (NT == 64) return v;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float total = red[0];
#pragma unroll
    for (int i = 1; i < NT / 64; ++i) total = fmaxf(total, red[i]);
    return total;
}
