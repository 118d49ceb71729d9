// RMSNorm over the float32 residual stream, with the residual sum fused in.
//
// Reference: somi_inference/models/qwen2.py:55-62
//   x32 = float(x); var = mean(x32^2); x32 = x32 * rsqrt(var + eps); y = w * cast(x32, in_dtype)
// Here the residual stream is float32 in both engines, square/mean/rsqrt/scale
// are float32, and the result is rounded once to the compute dtype (the
// reference rounds before the multiply by w when it runs in half precision).
#include "common.h"

// One workgroup per row.  ADD: h[row] += delta[row] first (and h is written back).
template <typename TO, typename TD, bool ADD>
__global__ void __launch_bounds__(256)
rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, const float* __restrict__ w, float eps,
               TO* __restrict__ out, int hidden) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float* hr = h + row * hidden;
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += 256) {
        float v = hr[i];
        if (ADD) {
            v += to_float(delta[row * hidden + i]);
            hr[i] = v;
        }
        ss += v * v;
    }
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
    TO* o = out + row * hidden;
    for (int i = threadIdx.x; i < hidden; i += 256) o[i] = from_float<TO>(w[i] * (hr[i] * inv));
}

// The same for widths that are a multiple of 4 up to 8192: a thread keeps its elements in registers
// (one pass over memory) and moves four at a time.
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

__device__ __forceinline__ f32x4 load4f(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load4f(const bf16* p) {
    const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
    return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
__device__ __forceinline__ void store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, f32x4 v) {
    *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
}

template <typename TO, typename TD, bool ADD, int CHUNKS>
__global__ void __launch_bounds__(256)
rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta, const float* __restrict__ w, float eps,
                   TO* __restrict__ out, int hidden) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float* hr = h + row * hidden;
    f32x4 v[CHUNKS];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = (c * 256 + threadIdx.x) * 4;
        v[c] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (i < hidden) {
            v[c] = load4f(hr + i);
            if (ADD) {
                v[c] += load4f(delta + row * hidden + i);
                store4(hr + i, v[c]);
            }
            ss += v[c][0] * v[c][0] + v[c][1] * v[c][1] + v[c][2] * v[c][2] + v[c][3] * v[c][3];
        }
    }
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = (c * 256 + threadIdx.x) * 4;
        if (i < hidden) {
            const f32x4 ww = load4f(w + i);
            store4(out + row * hidden + i, f32x4{ww[0] * (v[c][0] * inv), ww[1] * (v[c][1] * inv),
                                                 ww[2] * (v[c][2] * inv), ww[3] * (v[c][3] * inv)});
        }
    }
}

template <typename TO, typename TD, bool ADD>
static void launch_rmsnorm_vec(float* h, const void* delta, const float* w, float eps, void* out, int n, int hidden,
                               hipStream_t stream) {
    const int chunks = ceil_div(hidden, 1024);
#define SOMI_NORM(C)                                                                                          \
    hipLaunchKernelGGL((rmsnorm_vec_kernel<TO, TD, ADD, C>), dim3(n), dim3(256), 0, stream, h, (const TD*)delta, \
                       w, eps, (TO*)out, hidden)
    if (chunks <= 1) SOMI_NORM(1);
    else if (chunks <= 2) SOMI_NORM(2);
    else if (chunks <= 4) SOMI_NORM(4);
    else SOMI_NORM(8);
#undef SOMI_NORM
}

template <typename TO, typename TD>
static int launch_rmsnorm(float* h, const void* delta, const float* w, float eps, void* out, int n, int hidden,
                          hipStream_t stream) {
    const bool vec = hidden % 4 == 0 && hidden <= 8192 && (uintptr_t)h % 16 == 0 && (uintptr_t)w % 16 == 0 &&
                     (uintptr_t)out % 16 == 0 && (uintptr_t)delta % 16 == 0;
    if (vec) {
        if (delta) launch_rmsnorm_vec<TO, TD, true>(h, delta, w, eps, out, n, hidden, stream);
        else launch_rmsnorm_vec<TO, TD, false>(h, delta, w, eps, out, n, hidden, stream);
    } else if (delta)
        hipLaunchKernelGGL((rmsnorm_kernel<TO, TD, true>), dim3(n), dim3(256), 0, stream, h, (const TD*)delta, w,
                           eps, (TO*)out, hidden);
    else
        hipLaunchKernelGGL((rmsnorm_kernel<TO, TD, false>), dim3(n), dim3(256), 0, stream, h, (const TD*)nullptr,
                           w, eps, (TO*)out, hidden);
    SOMI_LAUNCH_CHECK("rmsnorm");
    return 0;
}

// h: [n, hidden] float32 (updated in place when delta is given); delta: [n, hidden] of dtype or null;
// w: [hidden] float32; out: [n, hidden] of dtype.
extern "C" int somi_rmsnorm(float* h, const void* delta, const float* w, float eps, void* out, int dtype, int n,
                            int hidden, hipStream_t stream) {
    SOMI_REQUIRE(n >= 0 && hidden > 0, "rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
    SOMI_REQUIRE(eps >= 0.f, "rmsnorm: eps must be >= 0, got %g", (double)eps);
    if (n == 0) return 0;
    if (dtype == SOMI_F32) return launch_rmsnorm<float, float>(h, delta, w, eps, out, n, hidden, stream);
    if (dtype == SOMI_BF16) return launch_rmsnorm<bf16, bf16>(h, delta, w, eps, out, n, hidden, stream);
    return somi_fail("rmsnorm: unknown dtype %d", dtype);
}

// h[i] += delta[i] in float32.
template <typename TD>
__global__ void __launch_bounds__(256)
residual_add_kernel(float* __restrict__ h, const TD* __restrict__ delta, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256)
        h[i] += to_float(delta[i]);
}

extern "C" int somi_residual_add(float* h, const void* delta, int dtype, int64_t count, hipStream_t stream) {
    SOMI_REQUIRE(count >= 0, "residual_add: bad count");
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(residual_add_kernel<float>, dim3(grid), dim3(256), 0, stream, h, (const float*)delta, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(residual_add_kernel<bf16>, dim3(grid), dim3(256), 0, stream, h, (const bf16*)delta, count);
    else
        return somi_fail("residual_add: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("residual_add");
    return 0;
}
