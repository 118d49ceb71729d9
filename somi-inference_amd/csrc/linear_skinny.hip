// Linear layer for few rows (decode): out[m, n] = sum_k x[m, k] * w[n, k] (+ bias[n]), bfloat16 in,
// float32 accumulation on the matrix cores, for M <= 64.
//
// Reference: the same nn.Linear products as linear_plain.hip (somi_inference/models/qwen2.py:221-222,
// 268-271; qwen2_adapter.py:60-62); the reference leaves them to a library.  With few rows the product
// is bound by reading w once from HBM, so the kernel is built around that stream:
//   * a workgroup owns 16 output columns (16 rows of w) and all rows of x; its WAVES wavefronts take
//     64-wide blocks of K in turn, so that at any time the workgroup reads WAVES * 128 contiguous bytes
//     of each of its 16 weight rows;
//   * a lane loads 2 x 16 bytes of one weight row and of one x row per block and issues two
//     v_mfma_f32_16x16x32_bf16 per 16 rows of x (w is the A operand, so a lane ends up with four
//     consecutive output columns of one row of x);
//   * the partial sums of the wavefronts are added through LDS in wavefront order, which fixes the
//     order of the additions whatever else runs.
// x is small and stays in L2; it is read directly.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <int MT, typename TO>
__global__ void __launch_bounds__(1024)
linear_skinny_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias,
                     TO* __restrict__ out, int M, int N, int K) {
    extern __shared__ float red[];                   // [waves][MT][64 lanes][4]
    const int waves = blockDim.x >> 6;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int wrow = (n0 + r < N) ? n0 + r : N - 1;
    const bf16* wp = w + (int64_t)wrow * K + g * 16;
    const bf16* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        xp[mt] = x + (int64_t)(m < M ? m : M - 1) * K + g * 16;
    }
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int stride = waves * 64;
    int k0 = wave * 64;
    for (; k0 + 64 <= K; k0 += stride) {             // whole blocks: no predicates
        const bf16x8 wa = load8(wp + k0), wb = load8(wp + k0 + 8);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const bf16x8 xa = load8(xp[mt] + k0), xb = load8(xp[mt] + k0 + 8);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xa, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, xb, acc[mt], 0, 0, 0);
        }
    }
    if (k0 < K) {                                    // the last, partial block (K is a multiple of 8)
        const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        const bool ha = k0 + g * 16 < K, hb = k0 + g * 16 + 8 < K;
        const bf16x8 wa = ha ? load8(wp + k0) : zero, wb = hb ? load8(wp + k0 + 8) : zero;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const bf16x8 xa = ha ? load8(xp[mt] + k0) : zero, xb = hb ? load8(xp[mt] + k0 + 8) : zero;
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xa, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, xb, acc[mt], 0, 0, 0);
        }
    }

#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
        *reinterpret_cast<f32x4*>(red + ((wave * MT + mt) * 64 + lane) * 4) = acc[mt];
    __syncthreads();
    for (int idx = threadIdx.x; idx < MT * 256; idx += blockDim.x) {
        float sum = 0.f;
        for (int wv = 0; wv < waves; ++wv) sum += red[wv * MT * 256 + idx];
        const int mt = idx >> 8, l = (idx >> 2) & 63, i = idx & 3;
        const int n = n0 + (l >> 4) * 4 + i;          // D[row = (lane / 16) * 4 + i][col = lane % 16]
        const int m = mt * 16 + (l & 15);
        if (n < N && m < M) {
            if (bias) sum += bias[n];
            out[(int64_t)m * N + n] = from_float<TO>(sum);
        }
    }
}

template <int MT, typename TO>
static int launch_skinny(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int waves,
                         hipStream_t stream) {
    const size_t smem = (size_t)waves * MT * 256 * sizeof(float);
    hipLaunchKernelGGL((linear_skinny_kernel<MT, TO>), dim3(ceil_div(N, 16)), dim3(waves * 64), smem, stream,
                       (const bf16*)x, (const bf16*)w, bias, (TO*)out, M, N, K);
    SOMI_LAUNCH_CHECK("linear_skinny");
    return 0;
}

// x: [M, K] bfloat16, w: [N, K] bfloat16, bias: [N] float32 or null, out: [M, N] bfloat16 or float32.
// M <= 64; K a multiple of 8; x and w 16-byte aligned.
extern "C" int somi_linear_skinny(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M,
                                  int N, int K, hipStream_t stream) {
    SOMI_REQUIRE(M >= 0 && N > 0 && K > 0, "linear_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
    SOMI_REQUIRE(M <= 64, "linear_skinny: at most 64 rows, got %d", M);
    SOMI_REQUIRE(K % 8 == 0, "linear_skinny: K (%d) must be a multiple of 8", K);
    SOMI_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "linear_skinny: x and w must be 16-byte aligned");
    SOMI_REQUIRE(out_dtype == SOMI_BF16 || out_dtype == SOMI_F32, "linear_skinny: unknown out dtype %d", out_dtype);
    if (M == 0) return 0;
    const int mt = ceil_div(M, 16);
    // Enough wavefronts to fill 256 compute units, at most 16 per workgroup, 64 KB of LDS, and no
    // more than there are 64-wide blocks of K.
    const int strips = ceil_div(N, 16);
    int waves = 16;
    while (waves > 4 && strips * (waves / 2) >= 4096) waves /= 2;
    while (waves > 1 && waves * mt > 32) waves /= 2;
    while (waves > 1 && waves * 64 > K + 63) waves /= 2;
#define SOMI_SKINNY(MT)                                                                                     \
    return out_dtype == SOMI_BF16 ? launch_skinny<MT, bf16>(x, w, bias, out, M, N, K, waves, stream)         \
                                  : launch_skinny<MT, float>(x, w, bias, out, M, N, K, waves, stream)
    switch (mt) {
        case 1: SOMI_SKINNY(1);
        case 2: SOMI_SKINNY(2);
        case 3: SOMI_SKINNY(3);
        default: SOMI_SKINNY(4);
    }
#undef SOMI_SKINNY
}
