// Plain linear layer: out[m, n] = sum_k x[m, k] * w[n, k] (+ bias[n]), float32 accumulation.
//
// Reference: nn.Linear / F.linear as used for q/k/v/o, the merged gate_up, down and the LM
// head (somi_inference/models/qwen2.py:221-222, 268-271, 296-298; qwen2_adapter.py:60-62).
// This is the true 32-bit path's matrix product (ordinary FMA, no reduced-precision matrix
// mode) and the reference the MFMA kernels are checked against.  Every output element is
// accumulated over k = 0..K-1 in order by one thread, so its value does not depend on how
// many rows the launch holds.
#include "common.h"

template <typename T, typename TO>
__global__ void __launch_bounds__(256)
linear_plain_kernel(const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ bias,
                    TO* __restrict__ out, int M, int N, int K) {
    __shared__ float As[16][68];   // [k][m]
    __shared__ float Bs[16][68];   // [k][n]
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = threadIdx.x + i * 256;
            const int r = idx >> 4, kk = idx & 15;
            const bool kin = (k0 + kk) < K;
            As[kk][r] = (kin && (m0 + r) < M) ? to_float(x[(int64_t)(m0 + r) * K + k0 + kk]) : 0.f;
            Bs[kk][r] = (kin && (n0 + r) < N) ? to_float(w[(int64_t)(n0 + r) * K + k0 + kk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += bias[n];
            out[(int64_t)m * N + n] = from_float<TO>(v);
        }
    }
}

// x: [M, K], w: [N, K] (row-major, as a checkpoint stores a linear layer), bias: [N] float32 or null,
// out: [M, N] of out_dtype (the input dtype, or float32 for logits).
extern "C" int somi_linear_plain(const void* x, const void* w, const float* bias, void* out, int dtype,
                                 int out_dtype, int M, int N, int K, hipStream_t stream) {
    SOMI_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    const dim3 grid(ceil_div(N, 64), ceil_div(M, 64));
    SOMI_REQUIRE(grid.y <= 65535, "linear: too many rows for one launch (M=%d)", M);
    if (dtype == SOMI_F32 && out_dtype == SOMI_F32)
        hipLaunchKernelGGL((linear_plain_kernel<float, float>), grid, dim3(256), 0, stream, (const float*)x,
                           (const float*)w, bias, (float*)out, M, N, K);
    else if (dtype == SOMI_BF16 && out_dtype == SOMI_BF16)
        hipLaunchKernelGGL((linear_plain_kernel<bf16, bf16>), grid, dim3(256), 0, stream, (const bf16*)x,
                           (const bf16*)w, bias, (bf16*)out, M, N, K);
    else if (dtype == SOMI_BF16 && out_dtype == SOMI_F32)
        hipLaunchKernelGGL((linear_plain_kernel<bf16, float>), grid, dim3(256), 0, stream, (const bf16*)x,
                           (const bf16*)w, bias, (float*)out, M, N, K);
    else
        return somi_fail("linear: unsupported dtypes in=%d out=%d", dtype, out_dtype);
    SOMI_LAUNCH_CHECK("linear_plain");
    return 0;
}
