// SwiGLU gate: out[t, i] = silu(gu[t, i]) * gu[t, I + i], silu(z) = z * sigmoid(z).
// Reference: somi_inference/models/qwen2.py:226-229 (chunk(2) of the merged projection, SiLU on the first half).
#include "common.h"

// block == 0: gu = [gate columns | up columns]; block == b > 0: gate and up columns interleaved in blocks of b
// (gate 0..b-1, up 0..b-1, gate b..2b-1, ...), the layout the fused decode kernel's weight has.
template <typename T>
__global__ void __launch_bounds__(256)
silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int block, int64_t count) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / inter;
        const int c = (int)(i - t * inter);
        const int at_gate = block > 0 ? (c / block) * 2 * block + c % block : c;
        const int at_up = block > 0 ? at_gate + block : inter + c;
        const float g = to_float(gu[t * 2 * inter + at_gate]);
        const float u = to_float(gu[t * 2 * inter + at_up]);
        const float s = g / (1.0f + expf(-g));
        out[i] = from_float<T>(s * u);
    }
}

// bfloat16, eight columns per thread (16-byte loads and stores); inter a multiple of 8 and, when
// interleaved, block a multiple of 8.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

__global__ void __launch_bounds__(256)
silu_mul_vec_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int inter, int block, int64_t groups) {
    const int per_row = inter / 8;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < groups; i += (int64_t)gridDim.x * 256) {
        const int64_t t = i / per_row;
        const int c = (int)(i - t * per_row) * 8;
        const int at_gate = block > 0 ? (c / block) * 2 * block + c % block : c;
        const int at_up = block > 0 ? at_gate + block : inter + c;
        const bf16x8 g = *reinterpret_cast<const bf16x8*>(gu + t * 2 * inter + at_gate);
        const bf16x8 u = *reinterpret_cast<const bf16x8*>(gu + t * 2 * inter + at_up);
        bf16x8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float gj = (float)g[j];
            o[j] = (bf16)(gj / (1.0f + expf(-gj)) * (float)u[j]);
        }
        *reinterpret_cast<bf16x8*>(out + t * inter + c) = o;
    }
}

extern "C" int somi_silu_mul(const void* gate_up, void* out, int dtype, int n_tokens, int inter, int block,
                             hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && inter > 0, "silu_mul: bad sizes n=%d inter=%d", n_tokens, inter);
    SOMI_REQUIRE(block >= 0 && (block == 0 || inter % block == 0), "silu_mul: block %d does not divide %d", block, inter);
    const int64_t count = (int64_t)n_tokens * inter;
    if (count == 0) return 0;
    const int grid = (int)(ceil_div64(count, 256) < 65536 ? ceil_div64(count, 256) : 65536);
    if (dtype == SOMI_BF16 && inter % 8 == 0 && (block == 0 || block % 8 == 0) && (uintptr_t)gate_up % 16 == 0 &&
        (uintptr_t)out % 16 == 0) {
        const int64_t groups = count / 8;
        const int vgrid = (int)(ceil_div64(groups, 256) < 65536 ? ceil_div64(groups, 256) : 65536);
        hipLaunchKernelGGL(silu_mul_vec_kernel, dim3(vgrid), dim3(256), 0, stream, (const bf16*)gate_up, (bf16*)out,
                           inter, block, groups);
        SOMI_LAUNCH_CHECK("silu_mul");
        return 0;
    }
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(silu_mul_kernel<float>, dim3(grid), dim3(256), 0, stream, (const float*)gate_up,
                           (float*)out, inter, block, count);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(silu_mul_kernel<bf16>, dim3(grid), dim3(256), 0, stream, (const bf16*)gate_up,
                           (bf16*)out, inter, block, count);
    else
        return somi_fail("silu_mul: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("silu_mul");
    return 0;
}
