// Linear layer for few rows (decode): out[m, n] = sum_k x[m, k] * w[n, k] (+ bias[n]), bfloat16 in,
// float32 accumulation on the matrix cores, for M <= 64.
//
// Reference: the same nn.Linear products as linear_plain.hip (somi_inference/models/qwen2.py:221-222,
// 268-271; qwen2_adapter.py:60-62); the reference leaves them to a library.  With few rows the product
// is bound by reading w once from HBM, so the kernel is built around that stream:
//   * a workgroup owns 16, 32 or 64 output columns (rows of w) and all rows of x; its wavefronts take
//     64-wide blocks of K in turn, so that at any time the workgroup reads (wavefronts * 128) contiguous
//     bytes of each of its weight rows;
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

template <int MT, int NS, int U, typename TO, bool SWIGLU>
__global__ void __launch_bounds__(1024)
linear_skinny_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias,
                     TO* __restrict__ out, int M, int N, int K) {
    extern __shared__ float red[];                   // [waves][NS][MT][64 lanes][4]
    const int waves = blockDim.x >> 6;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (16 * NS);
    const bf16* wp[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int row = n0 + s * 16 + r;
        wp[s] = w + (int64_t)(row < N ? row : N - 1) * K + g * 16;
    }
    const bf16* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        xp[mt] = x + (int64_t)(m < M ? m : M - 1) * K + g * 16;
    }
    f32x4 acc[NS][MT];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int stride = waves * 64;
    int k0 = wave * 64;
    // U whole blocks per trip: all their loads are issued before the first product
    for (; k0 + (U - 1) * stride + 64 <= K; k0 += U * stride) {
        bf16x8 wa[U][NS], wb[U][NS], xa[U][MT], xb[U][MT];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                wa[u][s] = load8(wp[s] + k0 + u * stride);
                wb[u][s] = load8(wp[s] + k0 + u * stride + 8);
            }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                xa[u][mt] = load8(xp[mt] + k0 + u * stride);
                xb[u][mt] = load8(xp[mt] + k0 + u * stride + 8);
            }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[u][s], xa[u][mt], acc[s][mt], 0, 0, 0);
                    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[u][s], xb[u][mt], acc[s][mt], 0, 0, 0);
                }
    }
    for (; k0 < K; k0 += stride) {                   // remaining blocks; the last may be partial (K % 8 == 0)
        const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        const bool ha = k0 + g * 16 < K, hb = k0 + g * 16 + 8 < K;
        bf16x8 xa[MT], xb[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            xa[mt] = ha ? load8(xp[mt] + k0) : zero;
            xb[mt] = hb ? load8(xp[mt] + k0 + 8) : zero;
        }
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const bf16x8 wa = ha ? load8(wp[s] + k0) : zero, wb = hb ? load8(wp[s] + k0 + 8) : zero;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xa[mt], acc[s][mt], 0, 0, 0);
                acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, xb[mt], acc[s][mt], 0, 0, 0);
            }
        }
    }

    constexpr int TILES = NS * MT;
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            *reinterpret_cast<f32x4*>(red + ((wave * TILES + s * MT + mt) * 64 + lane) * 4) = acc[s][mt];
    __syncthreads();
    if (SWIGLU) {
        // w holds gate and up rows interleaved in blocks of 16 (gate block j, up block j, gate block j + 1, ...):
        // strips 2p and 2p + 1 of this workgroup are gate and up of the same 16 output columns.
        const int n_out = N / 2;
        for (int idx = threadIdx.x; idx < (NS / 2) * MT * 256; idx += blockDim.x) {
            const int pair = idx / (MT * 256), rest = idx % (MT * 256);
            const int mt = rest >> 8, l = (rest >> 2) & 63, i = rest & 3;
            const int at_gate = ((2 * pair) * MT + mt) * 256 + (rest & 255);
            const int at_up = ((2 * pair + 1) * MT + mt) * 256 + (rest & 255);
            float gate = 0.f, up = 0.f;
            for (int wv = 0; wv < waves; ++wv) {
                gate += red[wv * TILES * 256 + at_gate];
                up += red[wv * TILES * 256 + at_up];
            }
            const int n = n0 / 2 + pair * 16 + (l >> 4) * 4 + i;
            const int m = mt * 16 + (l & 15);
            if (n < n_out && m < M) out[(int64_t)m * n_out + n] = from_float<TO>(gate / (1.0f + expf(-gate)) * up);
        }
        return;
    }
    for (int idx = threadIdx.x; idx < TILES * 256; idx += blockDim.x) {
        float sum = 0.f;
        for (int wv = 0; wv < waves; ++wv) sum += red[wv * TILES * 256 + idx];
        const int tile = idx >> 8, l = (idx >> 2) & 63, i = idx & 3;
        const int s = tile / MT, mt = tile % MT;
        const int n = n0 + s * 16 + (l >> 4) * 4 + i;          // D[row = (lane / 16) * 4 + i][col = lane % 16]
        const int m = mt * 16 + (l & 15);
        if (n < N && m < M) {
            if (bias) sum += bias[n];
            out[(int64_t)m * N + n] = from_float<TO>(sum);
        }
    }
}

template <int MT, int NS, int U, typename TO>
static int launch_skinny(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int waves,
                         bool swiglu, hipStream_t stream) {
    const size_t smem = (size_t)waves * NS * MT * 256 * sizeof(float);
    const dim3 grid(ceil_div(N, 16 * NS)), block(waves * 64);
    if (swiglu && NS >= 2)
        hipLaunchKernelGGL((linear_skinny_kernel<MT, (NS >= 2 ? NS : 2), U, TO, true>), grid, block, smem, stream,
                           (const bf16*)x, (const bf16*)w, bias, (TO*)out, M, N, K);
    else
        hipLaunchKernelGGL((linear_skinny_kernel<MT, NS, U, TO, false>), grid, block, smem, stream,
                           (const bf16*)x, (const bf16*)w, bias, (TO*)out, M, N, K);
    SOMI_LAUNCH_CHECK("linear_skinny");
    return 0;
}

template <int MT, int NS, typename TO>
static int launch_skinny_u(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                           int waves, int unroll, bool swiglu, hipStream_t stream) {
    if (NS * MT <= 4 && unroll >= 2)
        return launch_skinny<MT, NS, 2, TO>(x, w, bias, out, M, N, K, waves, swiglu, stream);
    return launch_skinny<MT, NS, 1, TO>(x, w, bias, out, M, N, K, waves, swiglu, stream);
}

template <int MT, typename TO>
static int launch_skinny_ns(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                            int waves, int strips, int unroll, bool swiglu, hipStream_t stream) {
    if (strips >= 4) return launch_skinny_u<MT, 4, TO>(x, w, bias, out, M, N, K, waves, unroll, swiglu, stream);
    if (strips >= 2) return launch_skinny_u<MT, 2, TO>(x, w, bias, out, M, N, K, waves, unroll, swiglu, stream);
    return launch_skinny_u<MT, 1, TO>(x, w, bias, out, M, N, K, waves, unroll, swiglu, stream);
}

static int skinny_dispatch(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M, int N,
                           int K, int waves, int strips, int unroll, bool swiglu, hipStream_t stream) {
    const int mt = ceil_div(M, 16);
#define SOMI_SKINNY(MT)                                                                                                  \
    return out_dtype == SOMI_BF16 ? launch_skinny_ns<MT, bf16>(x, w, bias, out, M, N, K, waves, strips, unroll, swiglu, stream)   \
                                  : launch_skinny_ns<MT, float>(x, w, bias, out, M, N, K, waves, strips, unroll, swiglu, stream)
    switch (mt) {
        case 1: SOMI_SKINNY(1);
        case 2: SOMI_SKINNY(2);
        case 3: SOMI_SKINNY(3);
        default: SOMI_SKINNY(4);
    }
#undef SOMI_SKINNY
}

static int skinny_check(const void* x, const void* w, int out_dtype, int M, int N, int K) {
    SOMI_REQUIRE(M >= 0 && N > 0 && K > 0, "linear_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
    SOMI_REQUIRE(M <= 64, "linear_skinny: at most 64 rows, got %d", M);
    SOMI_REQUIRE(K % 8 == 0, "linear_skinny: K (%d) must be a multiple of 8", K);
    SOMI_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "linear_skinny: x and w must be 16-byte aligned");
    SOMI_REQUIRE(out_dtype == SOMI_BF16 || out_dtype == SOMI_F32, "linear_skinny: unknown out dtype %d", out_dtype);
    return 0;
}

static int skinny_auto(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M, int N, int K,
                       bool swiglu, hipStream_t stream) {
    const int mt = ceil_div(M, 16);
    // Launch shape, from measurements at 7B layer sizes on MI355X.  x comes from L2 and its traffic, not
    // the weight stream, limits the kernel once there are several rows: then a wavefront computes 4
    // blocks of 16 columns from one read of x wherever that still leaves two workgroups per compute
    // unit.  One row is fastest with the widest split of K (16 wavefronts on one block of columns).
    const int blocks16 = ceil_div(N, 16);
    int strips = swiglu ? 2 : 1, waves = 16, unroll = 1;
    if (M > 1) {
        if (blocks16 >= 2048) {
            strips = 4;
            waves = blocks16 / 4 >= 1024 ? 8 : 4;
            unroll = 2;
        } else {
            waves = 8;
        }
    }
    while (waves > 1 && waves * mt * strips > 32) waves /= 2;      // 32 KB of LDS for the partial sums
    while (waves > 1 && waves * 64 > K + 63) waves /= 2;           // no more wavefronts than blocks of K
    if (K / (waves * 64) < 2) unroll = 1;
    return skinny_dispatch(x, w, bias, out, out_dtype, M, N, K, waves, strips, unroll, swiglu, stream);
}

// x: [M, K] bfloat16, w: [N, K] bfloat16, bias: [N] float32 or null, out: [M, N] bfloat16 or float32.
// M <= 64; K a multiple of 8; x and w 16-byte aligned.
extern "C" int somi_linear_skinny(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M,
                                  int N, int K, hipStream_t stream) {
    if (skinny_check(x, w, out_dtype, M, N, K)) return 1;
    if (M == 0) return 0;
    return skinny_auto(x, w, bias, out, out_dtype, M, N, K, false, stream);
}

// The gated feed-forward's first product with the gate fused in: w: [2 I, K] holds gate and up rows
// interleaved in blocks of 16 rows (gate rows 0..15, up rows 0..15, gate rows 16..31, ...); out: [M, I] with
// out[m, i] = silu(x . gate_i) * (x . up_i).  I must be a multiple of 16.
extern "C" int somi_linear_skinny_swiglu(const void* x, const void* w, void* out, int out_dtype, int M, int I, int K,
                                         hipStream_t stream) {
    if (skinny_check(x, w, out_dtype, M, 2 * I, K)) return 1;
    SOMI_REQUIRE(I % 16 == 0, "linear_skinny_swiglu: the intermediate size %d must be a multiple of 16", I);
    if (M == 0) return 0;
    return skinny_auto(x, w, nullptr, out, out_dtype, M, 2 * I, K, true, stream);
}

// The same product with the launch shape given by the caller (wavefronts per workgroup, 16-column
// strips per wavefront: 1, 2 or 4, unroll depth: 1 or 2): for measuring how the shape should be chosen.
extern "C" int somi_linear_skinny_shaped(const void* x, const void* w, const float* bias, void* out, int out_dtype,
                                         int M, int N, int K, int waves, int strips, int unroll, hipStream_t stream) {
    if (skinny_check(x, w, out_dtype, M, N, K)) return 1;
    SOMI_REQUIRE(strips == 1 || strips == 2 || strips == 4, "linear_skinny: strips must be 1, 2 or 4");
    SOMI_REQUIRE(waves >= 1 && waves <= 16 && waves * ceil_div(M, 16) * strips <= 32,
                 "linear_skinny: bad wavefront count %d", waves);
    if (M == 0) return 0;
    return skinny_dispatch(x, w, bias, out, out_dtype, M, N, K, waves, strips, unroll, false, stream);
}
