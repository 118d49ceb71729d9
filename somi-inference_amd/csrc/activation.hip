// SwiGLU gate: out[t, i] = silu(gu[t, i]) * gu[t, I + i], silu(z) = z * sigmoid(z).
// Reference: somi_inference/models/qwen2.py:226-229 (chunk(2) of the merged projection, SiLU on the first half).
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / inter;
        const int c = (int)(i - t * inter);
        const float g = to_float(gu[t * 2 * inter + c]);
        const float u = to_float(gu[t * 2 * inter + inter + c]);
        const float s = g / (1.0f + expf(-g));
        out[i] = from_float<T>(s * u);
    }
}

extern "C" int somi_silu_mul(const void* gate_up, void* out, int dtype, int n_tokens, int inter,
                             hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && inter > 0, "silu_mul: bad sizes n=%d inter=%d", n_tokens, inter);
    const int64_t count = (int64_t)n_tokens * inter;
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(silu_mul_kernel<float>, dim3(grid), dim3(256), 0, stream, (const float*)gate_up,
                           (float*)out, inter, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(silu_mul_kernel<bf16>, dim3(grid), dim3(256), 0, stream, (const bf16*)gate_up,
                           (bf16*)out, inter, count);
    else
        return somi_fail("silu_mul: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("silu_mul");
    return 0;
}
