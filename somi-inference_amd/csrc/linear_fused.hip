// Two forms of the few-rows product of linear_skinny.hip (at most 16 rows) that take the RMSNorm and the
// residual add of a pre-norm block into the products around them, so that a decode step launches no
// kernel of its own for either.  RMSNorm is weight * h * s with one scale s = 1 / sqrt(mean(h^2) + eps) per
// row, and a product is linear in that scale: norm(h) . W^T = s * ((weight * h) . W^T).  So
//
//   * the product INTO the residual stream (o_proj, down_proj):  h[m, n] += x[m, :] . w[n, :] (+ bias[n]) in
//     float32; the workgroup also writes the rows the next product reads, x'[m, n] = bfloat16(weight[n] *
//     h[m, n]) with the next norm's weight (no scale yet), and, for each row, the sum of squares of the new h
//     over its columns (`stats`: [workgroups][16] float32);
//   * the product OUT OF the residual stream (q/k/v, gate_up):  out = s * (x' . w^T) (+ bias), where s comes
//     from the producer's partial sums, added in workgroup order (a fixed order), and is applied to the
//     float32 sums (before the bias, before SiLU in the gated form).
//
// Against norm.hip the only difference is where the rounding to bfloat16 happens: on weight * h instead
// of weight * h * s (the same relative error; bfloat16 has float32's range, so the unscaled rows fit).
//
// Reference: somi_inference/models/qwen2.py:55-62 (RMSNorm), :333-339 (h = h + attn(norm(h)); h = h +
// mlp(norm(h))), :209-229 (gate_up with SiLU).  The streaming of w (coalesced buffer loads, two chunks in
// flight, a wavefront-private swizzled LDS tile, K split over the wavefronts, sums joined through LDS in
// wavefront order) is that of linear_skinny.hip.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

#define SOMI_BUFFER_WORD3 0x00020000u            // raw buffer, 32-bit elements, no swizzle
#define SOMI_OUT_OF_RANGE 0x80000000u
#define FUSED_MAX_WAVES 8
#define FUSED_CK 64
#define FUSED_SCALED 1
#define FUSED_RESIDUAL 2

template <int NS, int MODE, typename TO, bool SWIGLU, bool TAIL>
__global__ void __launch_bounds__(FUSED_MAX_WAVES * 64)
linear_fused_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias,
                    TO* __restrict__ out, float* __restrict__ h, const float* __restrict__ norm_w, float eps,
                    const float* __restrict__ stats_in, int stats_blocks, float* __restrict__ stats_out,
                    bf16* __restrict__ xnext, int M, int N, int K) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    __shared__ float row_scale[16];
    constexpr bool SCALED = MODE == FUSED_SCALED;
    constexpr int ROW_BYTES = FUSED_CK * 2;        // a row of a chunk in LDS: 64 bfloat16
    constexpr int WL = 2;                          // loads per 16 rows of w: 8 lanes read the 128 bytes of a row
    constexpr int XL = 2;                          // loads of the 16 rows of x
    constexpr int WAVE_BYTES = 16 * (NS + 1) * ROW_BYTES;
    constexpr int NW = NS * WL;

    const int waves = blockDim.x >> 6;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (16 * NS);
    char* mine = lds + wave * WAVE_BYTES;

    const int rows_here = min(16 * NS, N - n0);
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(w + (int64_t)n0 * K), 0, (int)((int64_t)rows_here * K * 2), SOMI_BUFFER_WORD3);
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(
        (void*)x, 0, (int)((int64_t)M * K * 2), SOMI_BUFFER_WORD3);

    auto swizzle = [](int row16) { return (row16 & 7) ^ (row16 >> 3); };
    // lane l reads 16 bytes (8 values) of row (l / 8) of each group of 8 rows
    const int lchunk = lane & 7;
    unsigned wgoff[NW];
    int wsoff[NW];
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        const int row16 = (i % WL) * 8 + (lane >> 3), tile = i / WL;
        wgoff[i] = ((unsigned)(tile * 16 + row16) * (unsigned)K + lchunk * 8) * 2u;
        wsoff[i] = (tile * 16 + row16) * ROW_BYTES + ((lchunk ^ swizzle(row16)) << 4);
    }
    unsigned xgoff[XL];
    int xsoff[XL];
#pragma unroll
    for (int j = 0; j < XL; ++j) {
        const int row16 = j * 8 + (lane >> 3);
        xgoff[j] = ((unsigned)row16 * (unsigned)K + lchunk * 8) * 2u;
        xsoff[j] = (NS * 16 + row16) * ROW_BYTES + ((lchunk ^ swizzle(row16)) << 4);
    }
    const int rswz = swizzle(r);

    f32x4 acc[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int chunks = (K + FUSED_CK - 1) / FUSED_CK;
    const int mine_n = wave < chunks ? (chunks - wave + waves - 1) / waves : 0;

    struct Stage {
        u32x4 wv[NW];
        u32x4 xv[XL];
    };
    auto issue = [&](Stage& st, int at) {
        const int k0 = (wave + at * waves) * FUSED_CK;
        const bool inside = !TAIL || k0 + lchunk * 8 < K;
#pragma unroll
        for (int i = 0; i < NW; ++i)
            st.wv[i] = __builtin_amdgcn_raw_buffer_load_b128(
                wres, inside ? wgoff[i] + (unsigned)k0 * 2u : SOMI_OUT_OF_RANGE, 0, 0);
#pragma unroll
        for (int j = 0; j < XL; ++j)
            st.xv[j] = __builtin_amdgcn_raw_buffer_load_b128(
                xres, inside ? xgoff[j] + (unsigned)k0 * 2u : SOMI_OUT_OF_RANGE, 0, 0);
    };
    auto stash = [&](const Stage& st) {
#pragma unroll
        for (int i = 0; i < NW; ++i) *reinterpret_cast<u32x4*>(mine + wsoff[i]) = st.wv[i];
#pragma unroll
        for (int j = 0; j < XL; ++j) *reinterpret_cast<u32x4*>(mine + xsoff[j]) = st.xv[j];
    };
    auto operand = [&](int tile, int c) -> bf16x8 {
        return *reinterpret_cast<const bf16x8*>(mine + (tile * 16 + r) * ROW_BYTES + ((c ^ rswz) << 4));
    };
    auto compute = [&]() {
        const bf16x8 xa = operand(NS, 2 * g), xb = operand(NS, 2 * g + 1);
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const bf16x8 wa = operand(s, 2 * g), wb = operand(s, 2 * g + 1);
            acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xa, acc[s], 0, 0, 0);
            acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, xb, acc[s], 0, 0, 0);
        }
    };

    // two chunks in flight
    Stage A, B;
    if (mine_n >= 1) issue(A, 0);                    // the first loads are under way while the scales are worked out
    if (mine_n >= 2) issue(B, 1);
    // The rows' scales come from the producer's partial sums of squares, added in a fixed order: thread t
    // adds the workgroups t / 16, t / 16 + threads / 16, ... of row t % 16, then 16 threads add those in thread
    // order.  The first loads go out here, before the weight stream, and are only looked at after it.
    constexpr int EARLY = 8;
    float early[EARLY];
    const int stride_b = blockDim.x >> 4;
    if (SCALED) {
#pragma unroll
        for (int i = 0; i < EARLY; ++i) {
            const int b = (threadIdx.x >> 4) + i * stride_b;
            early[i] = b < stats_blocks ? stats_in[b * 16 + (threadIdx.x & 15)] : 0.f;
        }
    }
    // the product into the stream: this thread's element of h, fetched ahead of its use in the epilogue
    const bool one_pass = (int)blockDim.x >= NS * 256;
    float h_before = 0.f;
    if (MODE == FUSED_RESIDUAL && one_pass && (int)threadIdx.x < NS * 256) {
        const int idx = threadIdx.x, l = (idx >> 2) & 63;
        const int n = n0 + (idx >> 8) * 16 + (l >> 4) * 4 + (idx & 3), m = l & 15;
        if (n < N && m < M) h_before = h[(int64_t)m * N + n];
    }

    if (mine_n >= 2) {
        int at = 0;
        for (; at + 3 < mine_n; at += 2) {
            stash(A);
            issue(A, at + 2);
            compute();
            stash(B);
            issue(B, at + 3);
            compute();
        }
        const bool third = at + 2 < mine_n;
        stash(A);
        if (third) issue(A, at + 2);
        compute();
        stash(B);
        compute();
        if (third) {
            stash(A);
            compute();
        }
    } else if (mine_n == 1) {
        stash(A);
        compute();
    }

    __shared__ float part[FUSED_MAX_WAVES * 64];
    if (SCALED) {
        float mine_sum = 0.f;
#pragma unroll
        for (int i = 0; i < EARLY; ++i) mine_sum += early[i];
        for (int b = (threadIdx.x >> 4) + EARLY * stride_b; b < stats_blocks; b += stride_b)
            mine_sum += stats_in[b * 16 + (threadIdx.x & 15)];
        part[threadIdx.x] = mine_sum;
    }
    __syncthreads();                                 // every wavefront is done with its staging space
    float* red = reinterpret_cast<float*>(lds);      // [waves][NS][64 lanes][4]
#pragma unroll
    for (int s = 0; s < NS; ++s) *reinterpret_cast<f32x4*>(red + ((wave * NS + s) * 64 + lane) * 4) = acc[s];
    if (SCALED && threadIdx.x < 16) {
        float sum = 0.f;
        for (int i = threadIdx.x; i < (int)blockDim.x; i += 16) sum += part[i];
        row_scale[threadIdx.x] = 1.0f / sqrtf(sum / (float)K + eps);
    }
    __syncthreads();
    if (SWIGLU) {
        // gate and up rows interleaved in blocks of 16: strips 2p and 2p + 1 are gate and up of the same columns
        const int n_out = N / 2;
        for (int idx = threadIdx.x; idx < (NS / 2) * 256; idx += blockDim.x) {
            const int pair = idx >> 8, l = (idx >> 2) & 63, i = idx & 3;
            float gate = 0.f, up = 0.f;
            for (int wv = 0; wv < waves; ++wv) {
                gate += red[(wv * NS + 2 * pair) * 256 + (idx & 255)];
                up += red[(wv * NS + 2 * pair + 1) * 256 + (idx & 255)];
            }
            const int n = n0 / 2 + pair * 16 + (l >> 4) * 4 + i, m = l & 15;
            if (SCALED) {
                gate *= row_scale[m];
                up *= row_scale[m];
            }
            if (n < n_out && m < M) out[(int64_t)m * n_out + n] = from_float<TO>(gate / (1.0f + expf(-gate)) * up);
        }
        return;
    }
    // D[row = (lane / 16) * 4 + i][col = lane % 16]: element idx of strip s is column n0 + 16 s + (l / 16) * 4 + i
    // of row l % 16 of x
    for (int idx = threadIdx.x; idx < NS * 256; idx += blockDim.x) {
        float sum = 0.f;
        for (int wv = 0; wv < waves; ++wv) sum += red[wv * NS * 256 + idx];
        const int s = idx >> 8, l = (idx >> 2) & 63, i = idx & 3;
        const int n = n0 + s * 16 + (l >> 4) * 4 + i, m = l & 15;
        float square = 0.f;
        if (SCALED) sum *= row_scale[m];
        if (n < N && m < M) {
            if (bias) sum += bias[n];
            if (MODE == FUSED_RESIDUAL) {
                const float now = (one_pass ? h_before : h[(int64_t)m * N + n]) + sum;
                h[(int64_t)m * N + n] = now;
                if (xnext) xnext[(int64_t)m * N + n] = (bf16)(norm_w[n] * now);
                square = now * now;
            } else {
                out[(int64_t)m * N + n] = from_float<TO>(sum);
            }
        }
        if (MODE == FUSED_RESIDUAL) red[idx] = square;     // only this thread read red[idx] of wavefront 0
    }
    if (MODE == FUSED_RESIDUAL) {
        __syncthreads();
        if (threadIdx.x < 16) {                      // row m: its squares over the workgroup's columns, in column order
            const int m = threadIdx.x;
            float total = 0.f;
            for (int s = 0; s < NS; ++s)
                for (int gg = 0; gg < 4; ++gg)
                    for (int i = 0; i < 4; ++i) total += red[s * 256 + (gg * 16 + m) * 4 + i];
            stats_out[blockIdx.x * 16 + m] = total;
        }
    }
}

static size_t fused_lds(int strips, int waves) {
    const size_t staging = (size_t)16 * (strips + 1) * FUSED_CK * 2, sums = (size_t)strips * 1024;
    return waves * (staging > sums ? staging : sums);
}

// The launch shape is linear_skinny.hip's for at most 16 rows: 8 wavefronts split K, two strips per
// workgroup where that leaves a workgroup for most compute units (one for very few rows and very many columns).
static int fused_strips(int M, int N, bool swiglu) {
    const int blocks16 = ceil_div(N, 16);
    int strips = 1;
    if (blocks16 >= 256) strips = 2;
    if (blocks16 >= 2048 && M <= 4) strips = 1;
    if (swiglu && strips < 2) strips = 2;
    return strips;
}

static int fused_waves(int K) {
    int waves = FUSED_MAX_WAVES;
    while (waves > 1 && waves * 64 > K + 63) waves /= 2;
    return waves;
}

template <int NS, int MODE, typename TO, bool SW>
static int fused_launch(const void* x, const void* w, const float* bias, void* out, float* h, const float* norm_w,
                        float eps, const float* stats_in, int stats_blocks, float* stats_out, void* xnext, int M, int N,
                        int K, hipStream_t stream) {
    const int waves = fused_waves(K);
    const dim3 grid(ceil_div(N, 16 * NS)), block(waves * 64);
    const size_t smem = fused_lds(NS, waves);
    if (K % FUSED_CK != 0)
        hipLaunchKernelGGL((linear_fused_kernel<NS, MODE, TO, SW, true>), grid, block, smem, stream, (const bf16*)x,
                           (const bf16*)w, bias, (TO*)out, h, norm_w, eps, stats_in, stats_blocks, stats_out, (bf16*)xnext,
                           M, N, K);
    else
        hipLaunchKernelGGL((linear_fused_kernel<NS, MODE, TO, SW, false>), grid, block, smem, stream, (const bf16*)x,
                           (const bf16*)w, bias, (TO*)out, h, norm_w, eps, stats_in, stats_blocks, stats_out, (bf16*)xnext,
                           M, N, K);
    SOMI_LAUNCH_CHECK("linear_fused");
    return 0;
}

static int fused_check(const void* x, const void* w, int M, int N, int K) {
    SOMI_REQUIRE(M >= 0 && N > 0 && K > 0, "linear_fused: bad sizes M=%d N=%d K=%d", M, N, K);
    SOMI_REQUIRE(M <= 16, "linear_fused: at most 16 rows, got %d", M);
    SOMI_REQUIRE(K % 8 == 0, "linear_fused: K (%d) must be a multiple of 8", K);
    SOMI_REQUIRE((int64_t)K * 4 * 64 < (int64_t)1 << 31, "linear_fused: K (%d) is too large", K);
    SOMI_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "linear_fused: x and w must be 16-byte aligned");
    return 0;
}

// Workgroups (= rows of the statistics) that somi_linear_residual launches for these sizes.
extern "C" int somi_linear_residual_blocks(int M, int N) { return ceil_div(N, 16 * fused_strips(M, N, false)); }

// h[m, n] += x[m, :] . w[n, :] (+ bias[n]).  x: [M, K] bfloat16; w: [N, K] bfloat16; bias: [N] float32 or null;
// h: [M, N] float32, in and out; stats: [somi_linear_residual_blocks(M, N)][16] float32, out: per workgroup and
// row the sum of squares of the new h over the workgroup's columns (rows M..15: 0); xnext: [M, N] bfloat16, out,
// = norm_w[n] * h[m, n] (norm_w: [N] float32), or null.  M <= 16.
extern "C" int somi_linear_residual(const void* x, const void* w, const float* bias, float* h, float* stats,
                                    const float* norm_w, void* xnext, int M, int N, int K, hipStream_t stream) {
    if (fused_check(x, w, M, N, K)) return 1;
    SOMI_REQUIRE(h && stats, "linear_residual: h and stats are needed");
    SOMI_REQUIRE(!xnext || norm_w, "linear_residual: the next rows need the norm's weight");
    if (M == 0) return 0;
    if (fused_strips(M, N, false) >= 2)
        return fused_launch<2, FUSED_RESIDUAL, float, false>(x, w, bias, nullptr, h, norm_w, 0.f, nullptr, 0, stats, xnext, M, N, K, stream);
    return fused_launch<1, FUSED_RESIDUAL, float, false>(x, w, bias, nullptr, h, norm_w, 0.f, nullptr, 0, stats, xnext, M, N, K, stream);
}

// out = s * (x . w^T) (+ bias) with the row scales s[m] = 1 / sqrt(sum of stats[:, m] / K + eps), or with swiglu
// (w: [2 I, K], gate and up rows interleaved in blocks of 16, no bias) out[m, i] = silu(s g) * (s u) for the gate
// and up products g, u.  x: [M, K] bfloat16, the rows somi_linear_residual wrote as xnext; stats:
// [stats_blocks][16] float32 from the same call; out: bfloat16.  M <= 16.
extern "C" int somi_linear_scaled(const void* x, float eps, const float* stats, int stats_blocks, const void* w,
                                  const float* bias, void* out, int M, int N, int K, int swiglu, hipStream_t stream) {
    if (fused_check(x, w, M, N, K)) return 1;
    SOMI_REQUIRE(stats && stats_blocks > 0, "linear_scaled: the row statistics are needed");
    SOMI_REQUIRE(!swiglu || (N % 32 == 0 && bias == nullptr), "linear_scaled: the gated form needs whole pairs of strips and no bias");
    if (M == 0) return 0;
    const int strips = fused_strips(M, N, swiglu != 0);
    if (swiglu)
        return fused_launch<2, FUSED_SCALED, bf16, true>(x, w, bias, out, nullptr, nullptr, eps, stats, stats_blocks, nullptr, nullptr, M, N, K, stream);
    if (strips >= 2)
        return fused_launch<2, FUSED_SCALED, bf16, false>(x, w, bias, out, nullptr, nullptr, eps, stats, stats_blocks, nullptr, nullptr, M, N, K, stream);
    return fused_launch<1, FUSED_SCALED, bf16, false>(x, w, bias, out, nullptr, nullptr, eps, stats, stats_blocks, nullptr, nullptr, M, N, K, stream);
}
