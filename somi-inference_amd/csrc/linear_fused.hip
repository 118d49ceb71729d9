// Two forms of the few-rows product of linear_skinny.hip (at most 64 rows) that take the RMSNorm and the
// residual add of a pre-norm block into the products around them, so that a decode step launches no
// kernel of its own for either.  RMSNorm is weight * h * s with one scale s = 1 / sqrt(mean(h^2) + eps) per
// row, and a product is linear in that scale: norm(h) . W^T = s * ((weight * h) . W^T).  So
//
//   * the product INTO the residual stream (o_proj, down_proj):  h[m, n] += x[m, :] . w[n, :] (+ bias[n]) in
//     float32; the workgroup also writes the rows the next product reads, x'[m, n] = bfloat16(weight[n] *
//     h[m, n]) with the next norm's weight (no scale yet), and, for each row, the sum of squares of the new h
//     over its columns (`stats`: [workgroups][16 * ceil(M / 16)] float32);
//   * the product OUT OF the residual stream (q/k/v, gate_up):  out = s * (x' . w^T) (+ bias), where s comes
//     from the producer's partial sums, added in workgroup order (a fixed order), and is applied to the
//     float32 sums (before the bias, before SiLU in the gated form).
//
// A third form is the q/k/v product whose end also applies the rotary position encoding to q and k and stores
// k and v in their cache pages (what rope_kv.hip does in a kernel of its own): a workgroup then owns the two
// 16-column strips of a head that are rotated together, columns j and j + D/2, instead of 32 neighbours.
//
// Against norm.hip the only difference is where the rounding to bfloat16 happens: on weight * h instead
// of weight * h * s (the same relative error; bfloat16 has float32's range, so the unscaled rows fit).
//
// Reference: somi_inference/models/qwen2.py:55-62 (RMSNorm), :333-339 (h = h + attn(norm(h)); h = h +
// mlp(norm(h))), :209-229 (gate_up with SiLU), :95-113 and :286-293 (rotation of q and k), core/paged_attention.py:
// 246-292 (k and v of a token land in its page).  The streaming of w (coalesced buffer loads, two chunks in
// flight, a wavefront-private swizzled LDS tile, K split over the wavefronts, sums joined through LDS in
// wavefront order) is that of linear_skinny.hip.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

#define SOMI_BUFFER_WORD3 0x00020000u            // raw buffer, 32-bit elements, no swizzle
#define SOMI_OUT_OF_RANGE 0x80000000u
#define FUSED_MAX_WAVES 8
#define FUSED_CK 64
#define FUSED_SCALED 1
#define FUSED_RESIDUAL 2

// What the q/k/v product needs to rotate q and k and to store k and v (the arguments of rope_kv.hip).
struct FusedRope {
    const int* positions;     // [M]
    const int* slots;         // [M]: page * page_size + offset of the token's k and v, or -1 for no store
    const float* inv_freq;    // [D / 2]
    bf16* k_cache;            // [pages, nkv, page_size, D]
    bf16* v_cache;            // [pages, nkv, D, page_size]
    int nq, nkv, D, page_size;
};

template <int MT, int NS, int MODE, typename TO, bool SWIGLU, bool TAIL, bool ROPE = false>
__global__ void __launch_bounds__(FUSED_MAX_WAVES * 64)
linear_fused_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias,
                    TO* __restrict__ out, float* __restrict__ h, const float* __restrict__ norm_w, float eps,
                    const float* __restrict__ stats_in, int stats_blocks, int stats_stride,
                    float* __restrict__ stats_out, bf16* __restrict__ xnext, int M, int N, int K, FusedRope rope) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    __shared__ float row_scale[64];
    __shared__ float part[FUSED_MAX_WAVES * 4 * 16 * MT];
    constexpr bool SCALED = MODE == FUSED_SCALED;
    constexpr int ROW_BYTES = FUSED_CK * 2;        // a row of a chunk in LDS: 64 bfloat16
    constexpr int ROWS = 16 * MT;                  // rows of x the kernel is built for
    constexpr int WAVE_BYTES = 16 * (NS + MT) * ROW_BYTES;
    constexpr int NL = (NS + MT) * 2;              // loads per lane and chunk: 8 lanes read the 128 bytes of a row
    constexpr int TILES = NS * MT;

    const int waves = blockDim.x >> 6;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = lane & 15, g = lane >> 4;
    // with the rotation, workgroup b owns the columns j .. j + 15 and j + D/2 .. of head b / (D / 32)
    const int rope_blocks = ROPE ? rope.D / 32 : 1;
    const int rope_head = blockIdx.x / rope_blocks, rope_j = (blockIdx.x % rope_blocks) * 16;
    const int n0 = ROPE ? rope_head * rope.D + rope_j : blockIdx.x * (16 * NS);
    const int strip_step = ROPE ? rope.D / 2 : 16;           // rows of w from one strip to the next
    char* mine = lds + wave * WAVE_BYTES;

    const int rows_here = ROPE ? N - n0 : min(16 * NS, N - n0);
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(w + (int64_t)n0 * K), 0, (int)((int64_t)rows_here * K * 2), SOMI_BUFFER_WORD3);
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(
        (void*)x, 0, (int)((int64_t)M * K * 2), SOMI_BUFFER_WORD3);

    auto swizzle = [](int row16) { return (row16 & 7) ^ (row16 >> 3); };
    // lane l reads 16 bytes (8 values) of row (l / 8) of each group of 8 rows; tiles 0..NS-1 are w, the others x
    const int lchunk = lane & 7;
    unsigned goff[NL];
    int soff[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int tile = i / 2, row16 = (i % 2) * 8 + (lane >> 3);
        const int row = tile < NS ? tile * strip_step + row16 : (tile - NS) * 16 + row16;
        goff[i] = ((unsigned)row * (unsigned)K + lchunk * 8) * 2u;
        soff[i] = (tile * 16 + row16) * ROW_BYTES + ((lchunk ^ swizzle(row16)) << 4);
    }
    const int rswz = swizzle(r);

    f32x4 acc[NS][MT];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int chunks = (K + FUSED_CK - 1) / FUSED_CK;
    const int mine_n = wave < chunks ? (chunks - wave + waves - 1) / waves : 0;

    auto issue = [&](u32x4 (&st)[NL], int at) {
        const int k0 = (wave + at * waves) * FUSED_CK;
        const bool inside = !TAIL || k0 + lchunk * 8 < K;
#pragma unroll
        for (int i = 0; i < NL; ++i)
            st[i] = i < NS * 2
                        ? __builtin_amdgcn_raw_buffer_load_b128(wres, inside ? goff[i] + (unsigned)k0 * 2u : SOMI_OUT_OF_RANGE, 0, SOMI_LOAD_ONCE)
                        : __builtin_amdgcn_raw_buffer_load_b128(xres, inside ? goff[i] + (unsigned)k0 * 2u : SOMI_OUT_OF_RANGE, 0, 0);
    };
    auto stash = [&](const u32x4 (&st)[NL]) {
#pragma unroll
        for (int i = 0; i < NL; ++i) *reinterpret_cast<u32x4*>(mine + soff[i]) = st[i];
    };
    auto operand = [&](int tile, int c) -> bf16x8 {
        return *reinterpret_cast<const bf16x8*>(mine + (tile * 16 + r) * ROW_BYTES + ((c ^ rswz) << 4));
    };
    auto compute = [&]() {
        bf16x8 xa[MT], xb[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            xa[mt] = operand(NS + mt, 2 * g);
            xb[mt] = operand(NS + mt, 2 * g + 1);
        }
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const bf16x8 wa = operand(s, 2 * g), wb = operand(s, 2 * g + 1);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xa[mt], acc[s][mt], 0, 0, 0);
                acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, xb[mt], acc[s][mt], 0, 0, 0);
            }
        }
    };

    u32x4 A[NL], B[NL];
    if (mine_n >= 1) issue(A, 0);                    // the first loads are under way while what follows is fetched
    if (mine_n >= 2) issue(B, 1);
    // The rows' scales come from the producer's partial sums of squares [stats_blocks][ROWS] (stats_stride floats
    // from one workgroup's sums to the next: these rows may be some of the rows of a longer table), added in a fixed
    // order: lane l of wavefront v adds the rows MT (l % 16) .. + MT - 1 (one load) of the workgroups
    // 4 v + l / 16, that + 4 waves, ...; then a thread per row adds those sums in order.  The first loads go
    // out here, before the weight stream, and are only looked at after it.
    constexpr int EARLY = 8;
    float early[EARLY][MT];
    const int stats_group = wave * 4 + g, stats_groups = waves * 4;
    auto stats_load = [&](float (&to)[MT], int block) {
        const float* from = stats_in + (int64_t)block * stats_stride + r * MT;
        if (block < stats_blocks) {
            __builtin_memcpy(&to[0], __builtin_assume_aligned(from, MT == 3 ? 4 : 4 * MT), 4 * MT);
        } else {
#pragma unroll
            for (int j = 0; j < MT; ++j) to[j] = 0.f;
        }
    };
    if (SCALED) {
#pragma unroll
        for (int i = 0; i < EARLY; ++i) stats_load(early[i], stats_group + i * stats_groups);
    }
    // The end of the kernel deals the sums out four consecutive columns (one lane's share of a tile) to a thread;
    // they are one access where the row length and the addresses keep them aligned and inside together.
    const bool whole = (N & 3) == 0 && (((uintptr_t)bias | (uintptr_t)h | (uintptr_t)norm_w) & 15) == 0 &&
                       (((uintptr_t)xnext | (uintptr_t)out) & 7) == 0;
    auto load4 = [&](const float* from, int n) -> f32x4 {
        if (whole) return *reinterpret_cast<const f32x4*>(from);
        f32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = n + i < N ? from[i] : 0.f;
        return v;
    };
    // the product into the stream: this thread's elements of h, fetched ahead of their use
    const bool one_pass = (int)blockDim.x >= TILES * 64;
    f32x4 h_before = {0.f, 0.f, 0.f, 0.f};
    if (MODE == FUSED_RESIDUAL && one_pass && (int)threadIdx.x < TILES * 64) {
        const int tile = threadIdx.x >> 6;
        const int n = n0 + (tile / MT) * 16 + g * 4, m = (tile % MT) * 16 + r;
        if (n < N && m < M) h_before = load4(h + (int64_t)m * N + n, n);
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

    if (SCALED) {
        float mine_sum[MT];
#pragma unroll
        for (int j = 0; j < MT; ++j) mine_sum[j] = 0.f;
#pragma unroll
        for (int i = 0; i < EARLY; ++i)
#pragma unroll
            for (int j = 0; j < MT; ++j) mine_sum[j] += early[i][j];
        for (int b = stats_group + EARLY * stats_groups; b < stats_blocks; b += stats_groups) {
            float more[MT];
            stats_load(more, b);
#pragma unroll
            for (int j = 0; j < MT; ++j) mine_sum[j] += more[j];
        }
#pragma unroll
        for (int j = 0; j < MT; ++j) part[stats_group * ROWS + r * MT + j] = mine_sum[j];
    }
    __syncthreads();                                 // every wavefront is done with its staging space
    float* red = reinterpret_cast<float*>(lds);      // [waves][TILES][64 lanes][4]
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            *reinterpret_cast<f32x4*>(red + ((wave * TILES + s * MT + mt) * 64 + lane) * 4) = acc[s][mt];
    if (SCALED && threadIdx.x < ROWS) {
        float sum = 0.f;
        for (int group = 0; group < stats_groups; ++group) sum += part[group * ROWS + threadIdx.x];
        row_scale[threadIdx.x] = 1.0f / sqrtf(sum / (float)K + eps);
    }
    __syncthreads();
    if constexpr (ROPE) {
        // lane l of row tile mt holds the channels j .. j + 3 (j = rope_j + (l / 16) * 4) of row 16 mt + l % 16 in the
        // first strip and the channels they are rotated with, j + D/2 .., in the second
        const int D = rope.D, nq = rope.nq, nkv = rope.nkv;
        for (int item = threadIdx.x; item < MT * 64; item += blockDim.x) {
            const int mt = item >> 6, l = item & 63, m = mt * 16 + (l & 15), j = rope_j + (l >> 4) * 4;
            f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = lo;
            for (int wv = 0; wv < waves; ++wv) {
                lo += *reinterpret_cast<const f32x4*>(red + ((wv * TILES + mt) * 64 + l) * 4);
                hi += *reinterpret_cast<const f32x4*>(red + ((wv * TILES + MT + mt) * 64 + l) * 4);
            }
            if (m >= M) continue;
            if (SCALED) {
                lo *= row_scale[m];
                hi *= row_scale[m];
            }
            if (bias) {
                lo += load4(bias + rope_head * D + j, 0);
                hi += load4(bias + rope_head * D + D / 2 + j, 0);
            }
            bf16x4 first, second;
            if (rope_head < nq + nkv) {                    // q and k heads: x' = x cos + rotate_half(x) sin
                const float pos = (float)rope.positions[m];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // the product is rounded to bfloat16 before it is rotated, as where the rotation is a kernel
                    // of its own: k in the cache does not depend on which of the two wrote it
                    const float x1 = to_float((bf16)lo[i]), x2 = to_float((bf16)hi[i]);
                    const float angle = pos * rope.inv_freq[j + i];
                    const float c = cosf(angle), sn = sinf(angle);
                    first[i] = (bf16)(x1 * c - x2 * sn);
                    second[i] = (bf16)(x2 * c + x1 * sn);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    first[i] = (bf16)lo[i];
                    second[i] = (bf16)hi[i];
                }
            }
            if (rope_head < nq) {
                bf16* to = reinterpret_cast<bf16*>(out) + (int64_t)m * nq * D + rope_head * D + j;
                *reinterpret_cast<bf16x4*>(to) = first;
                *reinterpret_cast<bf16x4*>(to + D / 2) = second;
                continue;
            }
            const int slot = rope.slots[m];
            if (slot < 0) continue;
            const int64_t page = slot / rope.page_size, off = slot % rope.page_size;
            if (rope_head < nq + nkv) {
                bf16* to = rope.k_cache + ((page * nkv + (rope_head - nq)) * rope.page_size + off) * D + j;
                *reinterpret_cast<bf16x4*>(to) = first;
                *reinterpret_cast<bf16x4*>(to + D / 2) = second;
            } else {                                       // v is kept transposed inside a page
                bf16* to = rope.v_cache + ((page * nkv + (rope_head - nq - nkv)) * D + j) * rope.page_size + off;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    to[(int64_t)i * rope.page_size] = first[i];
                    to[(int64_t)(D / 2 + i) * rope.page_size] = second[i];
                }
            }
        }
        return;
    }
    if (SWIGLU) {
        // gate and up rows interleaved in blocks of 16: strips 2p and 2p + 1 are gate and up of the same columns
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
            const int n = n0 / 2 + pair * 16 + (l >> 4) * 4 + i, m = mt * 16 + (l & 15);
            if (SCALED) {
                gate *= row_scale[m];
                up *= row_scale[m];
            }
            if (n < n_out && m < M) out[(int64_t)m * n_out + n] = from_float<TO>(gate / (1.0f + expf(-gate)) * up);
        }
        return;
    }
    // D[row = (lane / 16) * 4 + i][col = lane % 16]: lane l of tile (s, mt) holds the columns
    // n0 + 16 s + (l / 16) * 4 .. + 3 of row 16 mt + l % 16 of x
    for (int item = threadIdx.x; item < TILES * 64; item += blockDim.x) {
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (int wv = 0; wv < waves; ++wv) sum += *reinterpret_cast<const f32x4*>(red + (wv * TILES * 64 + item) * 4);
        const int tile = item >> 6, l = item & 63;
        const int n = n0 + (tile / MT) * 16 + (l >> 4) * 4, m = (tile % MT) * 16 + (l & 15);
        float square = 0.f;
        if (SCALED) sum *= row_scale[m];
        if (n < N && m < M) {
            if (bias) sum += load4(bias + n, n);
            const int64_t at = (int64_t)m * N + n;
            if (MODE == FUSED_RESIDUAL) {
                const f32x4 now = (one_pass ? h_before : load4(h + at, n)) + sum;
                const f32x4 scaled = xnext ? load4(norm_w + n, n) * now : now;
                if (whole) {
                    *reinterpret_cast<f32x4*>(h + at) = now;
                    if (xnext) {
                        bf16x4 next;
#pragma unroll
                        for (int i = 0; i < 4; ++i) next[i] = (bf16)scaled[i];
                        *reinterpret_cast<bf16x4*>(xnext + at) = next;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (n + i >= N) continue;
                        h[at + i] = now[i];
                        if (xnext) xnext[at + i] = (bf16)scaled[i];
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) square += n + i < N ? now[i] * now[i] : 0.f;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) out[at + i] = from_float<TO>(sum[i]);
            }
        }
        if (MODE == FUSED_RESIDUAL) part[item] = square;
    }
    if (MODE == FUSED_RESIDUAL) {
        __syncthreads();
        if (threadIdx.x < ROWS) {                    // a row's squares over the workgroup's columns, in column order
            const int mt = threadIdx.x >> 4, rr = threadIdx.x & 15;
            float total = 0.f;
            for (int s = 0; s < NS; ++s)
                for (int gg = 0; gg < 4; ++gg) total += part[(s * MT + mt) * 64 + gg * 16 + rr];
            stats_out[(int64_t)blockIdx.x * stats_stride + threadIdx.x] = total;
        }
    }
}

static size_t fused_lds(int mt, int strips, int waves) {
    const size_t staging = (size_t)16 * (strips + mt) * FUSED_CK * 2, sums = (size_t)strips * mt * 1024;
    return waves * (staging > sums ? staging : sums);
}

// The launch shape is linear_skinny.hip's: 8 wavefronts split K; two strips per workgroup where that leaves a
// workgroup for most compute units (one for very few rows and very many columns).
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

template <int MT, int NS, int MODE, typename TO, bool SW, bool TL, bool ROPE>
static void fused_launch_kernel(const void* x, const void* w, const float* bias, void* out, float* h,
                                const float* norm_w, float eps, const float* stats_in, int stats_blocks,
                                int stats_stride, float* stats_out, void* xnext, int M, int N, int K,
                                const FusedRope& rope, hipStream_t stream) {
    const int waves = fused_waves(K);
    const dim3 grid(ROPE ? (rope.nq + 2 * rope.nkv) * (rope.D / 32) : ceil_div(N, 16 * NS)), block(waves * 64);
    const size_t smem = fused_lds(MT, NS, waves);
    if (smem > 64 * 1024)                            // beyond the default limit of dynamic LDS
        (void)hipFuncSetAttribute((const void*)linear_fused_kernel<MT, NS, MODE, TO, SW, TL, ROPE>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL((linear_fused_kernel<MT, NS, MODE, TO, SW, TL, ROPE>), grid, block, smem, stream,
                       (const bf16*)x, (const bf16*)w, bias, (TO*)out, h, norm_w, eps, stats_in, stats_blocks,
                       stats_stride > 0 ? stats_stride : 16 * MT, stats_out, (bf16*)xnext, M, N, K, rope);
}

template <int NS, int MODE, typename TO, bool SW, bool ROPE = false>
static int fused_launch(const void* x, const void* w, const float* bias, void* out, float* h, const float* norm_w,
                        float eps, const float* stats_in, int stats_blocks, float* stats_out, void* xnext, int M, int N,
                        int K, hipStream_t stream, const FusedRope& rope = FusedRope{}, int stats_stride = 0) {
    const bool tail = K % FUSED_CK != 0;
#define SOMI_FUSED(MT)                                                                                               \
    if (tail) fused_launch_kernel<MT, NS, MODE, TO, SW, true, ROPE>(x, w, bias, out, h, norm_w, eps, stats_in,          \
                                                                    stats_blocks, stats_stride, stats_out, xnext, M, \
                                                                    N, K, rope, stream);                              \
    else fused_launch_kernel<MT, NS, MODE, TO, SW, false, ROPE>(x, w, bias, out, h, norm_w, eps, stats_in,             \
                                                                stats_blocks, stats_stride, stats_out, xnext, M, N,  \
                                                                K, rope, stream);                                     \
    break
    switch (ceil_div(M, 16)) {
        case 1: SOMI_FUSED(1);
        case 2: SOMI_FUSED(2);
        case 3: SOMI_FUSED(3);
        default: SOMI_FUSED(4);
    }
#undef SOMI_FUSED
    SOMI_LAUNCH_CHECK("linear_fused");
    return 0;
}

static int fused_check(const void* x, const void* w, int M, int N, int K) {
    SOMI_REQUIRE(M >= 0 && N > 0 && K > 0, "linear_fused: bad sizes M=%d N=%d K=%d", M, N, K);
    SOMI_REQUIRE(M <= 64, "linear_fused: at most 64 rows, got %d", M);
    SOMI_REQUIRE(K % 8 == 0, "linear_fused: K (%d) must be a multiple of 8", K);
    SOMI_REQUIRE((int64_t)K * 2 * 64 < (int64_t)1 << 31, "linear_fused: K (%d) is too large", K);
    SOMI_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "linear_fused: x and w must be 16-byte aligned");
    return 0;
}

// Workgroups (= rows of the statistics) that somi_linear_residual launches for these sizes.
extern "C" int somi_linear_residual_blocks(int M, int N) { return ceil_div(N, 16 * fused_strips(M, N, false)); }

// h[m, n] += x[m, :] . w[n, :] (+ bias[n]).  x: [M, K] bfloat16; w: [N, K] bfloat16; bias: [N] float32 or null;
// h: [M, N] float32, in and out; stats: [somi_linear_residual_blocks(M, N)][16 ceil(M / 16)] float32, out: per
// workgroup and row the sum of squares of the new h over the workgroup's columns (rows from M on: 0); xnext:
// [M, N] bfloat16, out, = norm_w[n] * h[m, n] (norm_w: [N] float32), or null.  M <= 64.  stats_stride: floats from
// one workgroup's sums to the next where they are columns of the table of more rows (a multiple of 4), or 0.
extern "C" int somi_linear_residual(const void* x, const void* w, const float* bias, float* h, float* stats,
                                    int stats_stride, const float* norm_w, void* xnext, int M, int N, int K,
                                    hipStream_t stream) {
    if (fused_check(x, w, M, N, K)) return 1;
    SOMI_REQUIRE(h && stats, "linear_residual: h and stats are needed");
    SOMI_REQUIRE(!xnext || norm_w, "linear_residual: the next rows need the norm's weight");
    SOMI_REQUIRE(stats_stride == 0 || (stats_stride % 4 == 0 && stats_stride >= 16 * ceil_div(M, 16)),
                 "linear_residual: a stride of %d floats does not hold the sums of %d rows", stats_stride, M);
    if (M == 0) return 0;
    if (fused_strips(M, N, false) >= 2)
        return fused_launch<2, FUSED_RESIDUAL, float, false>(x, w, bias, nullptr, h, norm_w, 0.f, nullptr, 0, stats, xnext, M, N, K, stream, FusedRope{}, stats_stride);
    return fused_launch<1, FUSED_RESIDUAL, float, false>(x, w, bias, nullptr, h, norm_w, 0.f, nullptr, 0, stats, xnext, M, N, K, stream, FusedRope{}, stats_stride);
}

// out = s * (x . w^T) (+ bias) with the row scales s[m] = 1 / sqrt(sum of stats[:, m] / K + eps), or with swiglu
// (w: [2 I, K], gate and up rows interleaved in blocks of 16, no bias) out[m, i] = silu(s g) * (s u) for the gate
// and up products g, u.  x: [M, K] bfloat16, the rows a product into the stream wrote as xnext; stats:
// [stats_blocks][16 ceil(M / 16)] float32 from the same call; out: bfloat16.  M <= 64.
extern "C" int somi_linear_scaled(const void* x, float eps, const float* stats, int stats_blocks, const void* w,
                                  const float* bias, void* out, int M, int N, int K, int swiglu, hipStream_t stream) {
    if (fused_check(x, w, M, N, K)) return 1;
    SOMI_REQUIRE(stats && stats_blocks > 0 && (uintptr_t)stats % 16 == 0, "linear_scaled: the row statistics are needed, 16-byte aligned");
    SOMI_REQUIRE(!swiglu || (N % 32 == 0 && bias == nullptr), "linear_scaled: the gated form needs whole pairs of strips and no bias");
    if (M == 0) return 0;
    const int strips = fused_strips(M, N, swiglu != 0);
    if (swiglu)
        return fused_launch<2, FUSED_SCALED, bf16, true>(x, w, bias, out, nullptr, nullptr, eps, stats, stats_blocks, nullptr, nullptr, M, N, K, stream);
    if (strips >= 2)
        return fused_launch<2, FUSED_SCALED, bf16, false>(x, w, bias, out, nullptr, nullptr, eps, stats, stats_blocks, nullptr, nullptr, M, N, K, stream);
    return fused_launch<1, FUSED_SCALED, bf16, false>(x, w, bias, out, nullptr, nullptr, eps, stats, stats_blocks, nullptr, nullptr, M, N, K, stream);
}

// The q/k/v product with the rotary encoding and the cache store in its end.  x: [M, K] bfloat16; w:
// [(nq + 2 nkv) D, K] bfloat16, the rows of the q heads, then the k heads, then the v heads; bias: float32 or
// null.  With stats (from a product into the stream, see somi_linear_scaled) the sums are scaled per row
// first; with stats == null x is used as it is.  q: [M, nq D] bfloat16, out, rotated; k (rotated) and v go to
// their pages: k_cache [pages, nkv, page_size, D], v_cache [pages, nkv, D, page_size], slot of row m =
// page * page_size + offset or -1.  positions: [M] int32; inv_freq: [D / 2] float32 (the whole head is
// rotated).  D must be a multiple of 32, M <= 64.  stats_stride: floats from one workgroup's sums to the next where
// the M rows are some of the rows of a longer table (a multiple of 4), or 0 for 16 ceil(M / 16).
extern "C" int somi_linear_rope_store(const void* x, float eps, const float* stats, int stats_blocks, int stats_stride, const void* w,
                                      const float* bias, void* q, const int* positions, const int* slots,
                                      const float* inv_freq, void* k_cache, void* v_cache, int nq, int nkv, int D,
                                      int page_size, int M, int K, hipStream_t stream) {
    SOMI_REQUIRE(nq > 0 && nkv > 0 && D > 0 && D % 32 == 0, "linear_rope_store: head_dim (%d) must be a multiple of 32", D);
    const int64_t columns = (int64_t)(nq + 2 * nkv) * D;
    SOMI_REQUIRE(columns * K * 2 < (int64_t)1 << 31, "linear_rope_store: the weight is too large");
    const int N = (int)columns;
    if (fused_check(x, w, M, N, K)) return 1;
    SOMI_REQUIRE(q && positions && slots && inv_freq && k_cache && v_cache && page_size > 0,
                 "linear_rope_store: q, positions, slots, inv_freq and the caches are needed");
    SOMI_REQUIRE((uintptr_t)q % 8 == 0 && (uintptr_t)k_cache % 8 == 0, "linear_rope_store: q and the k cache must be 8-byte aligned");
    SOMI_REQUIRE(!stats || (stats_blocks > 0 && (uintptr_t)stats % 16 == 0), "linear_rope_store: bad row statistics");
    SOMI_REQUIRE(stats_stride == 0 || (stats_stride % 4 == 0 && stats_stride >= 16 * ceil_div(M, 16)),
                 "linear_rope_store: a stride of %d floats does not hold the sums of %d rows", stats_stride, M);
    if (M == 0) return 0;
    const FusedRope rope{positions, slots, inv_freq, (bf16*)k_cache, (bf16*)v_cache, nq, nkv, D, page_size};
    if (stats)
        return fused_launch<2, FUSED_SCALED, bf16, false, true>(x, w, bias, q, nullptr, nullptr, eps, stats, stats_blocks,
                                                                nullptr, nullptr, M, N, K, stream, rope, stats_stride);
    return fused_launch<2, 0, bf16, false, true>(x, w, bias, q, nullptr, nullptr, 0.f, nullptr, 0, nullptr, nullptr, M, N, K,
                                                 stream, rope);
}
