// Linear layer for few rows (decode): out[m, n] = sum_k x[m, k] * w[n, k] (+ bias[n]), bfloat16 in,
// float32 accumulation on the matrix cores, for M <= 64.
//
// Reference: the same nn.Linear products as linear_plain.hip (somi_inference/models/qwen2.py:221-222,
// 268-271; qwen2_adapter.py:60-62); the reference leaves them to a library.  With few rows the product
// is bound by reading w once from HBM, so the kernel is built around that stream.  The matrix core
// wants lane l to hold 8 k-values of row (l % 16); a load straight into that layout makes every
// group of four lanes touch four different rows (16 bytes from each of 64 places per instruction),
// which costs a fifth of the bandwidth.  Here a wavefront reads whole pieces of rows instead (8
// consecutive lanes read 128 consecutive bytes of one row, or 16 lanes 256 bytes), keeps DEPTH such
// chunks in flight in registers, and turns them through a private piece of LDS into the operand layout:
//   * a workgroup owns NS blocks of 16 output columns and all rows of x; its wavefronts take chunks
//     of CK values of K in turn; a chunk is the workgroup's 16 * NS rows of w and the rows of x;
//   * loads are buffer loads whose range ends at the last valid row, so rows past N or M read as zero
//     without a branch; a chunk that crosses K is masked per lane the same way;
//   * LDS rows are XOR-swizzled in 16-byte units so that neither the row-wise writes nor the
//     column-wise operand reads collide, whether 8 or 16 lanes are served per cycle;
//   * w is the A operand, so a lane ends up with four consecutive output columns of one row of x;
//   * partial sums of the wavefronts are added through LDS in wavefront order, which fixes the order
//     of the additions whatever else runs.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

#define SOMI_BUFFER_WORD3 0x00020000u            // raw buffer, 32-bit elements, no swizzle
#define SOMI_OUT_OF_RANGE 0x80000000u
#define SKINNY_MAX_WAVES 8

template <int MT, int NS, int CK, int DEPTH, typename TO, bool SWIGLU, bool TAIL>
__global__ void __launch_bounds__(SKINNY_MAX_WAVES * 64)
linear_skinny_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias,
                     TO* __restrict__ out, int M, int N, int K) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    constexpr int ROW_BYTES = CK * 2;              // bytes of one row in a chunk: 256 or 128
    constexpr int LPR = ROW_BYTES / 16;            // lanes that read one row: 16 or 8
    constexpr int RPI = 64 / LPR;                  // rows per load instruction: 4 or 8
    constexpr int WL = 16 / RPI;                   // load instructions per 16 rows: 4 or 2
    constexpr int ROWS = 16 * (NS + MT);
    constexpr int WAVE_BYTES = ROWS * ROW_BYTES;
    constexpr int NL = (NS + MT) * WL;             // loads per lane and chunk
    constexpr int TILES = NS * MT;

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

    // where this lane reads (bytes from the start of the workgroup's rows) and writes (bytes in LDS)
    const int lrow = lane / LPR, lchunk = lane % LPR;
    unsigned goff[NL];
    int soff[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int tile = i / WL, j = i % WL;       // tiles 0..NS-1 are w, the others are x
        const int row16 = j * RPI + lrow;          // row inside the tile
        const int row = tile < NS ? tile * 16 + row16 : (tile - NS) * 16 + row16;
        goff[i] = ((unsigned)row * (unsigned)K + lchunk * 8) * 2u;
        const int swz = CK == 128 ? (row16 & 15) : ((row16 & 7) ^ (row16 >> 3));
        soff[i] = (tile * 16 + row16) * ROW_BYTES + ((lchunk ^ swz) << 4);
    }
    const int rswz = CK == 128 ? r : ((r & 7) ^ (r >> 3));

    f32x4 acc[NS][MT];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int chunks = (K + CK - 1) / CK;
    const int mine_n = wave < chunks ? (chunks - wave + waves - 1) / waves : 0;

    auto issue = [&](u32x4 (&st)[NL], int at) {
        const int k0 = (wave + at * waves) * CK;
        const bool inside = !TAIL || k0 + lchunk * 8 < K;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const unsigned off = inside ? goff[i] + (unsigned)k0 * 2u : SOMI_OUT_OF_RANGE;
            st[i] = i < NS * WL ? __builtin_amdgcn_raw_buffer_load_b128(wres, off, 0, SOMI_LOAD_ONCE)
                                : __builtin_amdgcn_raw_buffer_load_b128(xres, off, 0, 0);
        }
    };
    auto stash = [&](const u32x4 (&st)[NL]) {
#pragma unroll
        for (int i = 0; i < NL; ++i) *reinterpret_cast<u32x4*>(mine + soff[i]) = st[i];
    };
    auto operand = [&](int tile, int c) -> bf16x8 {
        return *reinterpret_cast<const bf16x8*>(mine + (tile * 16 + r) * ROW_BYTES + ((c ^ rswz) << 4));
    };
    // the k-values of a 64-wide block are dealt to the two products as 16-byte pieces 2g and 2g + 1 of
    // lane group g: any order serves as long as w and x use the same
    auto compute = [&]() {
#pragma unroll
        for (int cb = 0; cb < CK / 64; ++cb) {
            bf16x8 xa[MT], xb[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                xa[mt] = operand(NS + mt, cb * 8 + 2 * g);
                xb[mt] = operand(NS + mt, cb * 8 + 2 * g + 1);
            }
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const bf16x8 wa = operand(s, cb * 8 + 2 * g), wb = operand(s, cb * 8 + 2 * g + 1);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xa[mt], acc[s][mt], 0, 0, 0);
                    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, xb[mt], acc[s][mt], 0, 0, 0);
                }
            }
        }
    };

    // DEPTH chunks in flight: set d holds chunk `at + d`.  The loop is entered on one path only, with
    // every set issued, so that the waits inside it count loads exactly.
    u32x4 st[DEPTH][NL];
    if (mine_n >= DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) issue(st[d], d);
        int at = 0;
        for (; at + 2 * DEPTH - 1 < mine_n; at += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                stash(st[d]);
                issue(st[d], at + DEPTH + d);
                compute();
            }
        }
        // DEPTH to 2 * DEPTH - 1 chunks are left
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            stash(st[d]);
            if (d < DEPTH - 1 && at + DEPTH + d < mine_n) issue(st[d], at + DEPTH + d);
            compute();
        }
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (at + DEPTH + d < mine_n) {
                stash(st[d]);
                compute();
            }
    } else {
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (d < mine_n) issue(st[d], d);
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (d < mine_n) {
                stash(st[d]);
                compute();
            }
    }

    __syncthreads();                                 // every wavefront is done with its staging space
    float* red = reinterpret_cast<float*>(lds);      // [waves][TILES][64 lanes][4]
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

// LDS of a launch: the staging space of every wavefront, or the partial sums, whichever is larger.
static size_t skinny_lds(int mt, int strips, int chunk, int waves) {
    const size_t staging = (size_t)16 * (strips + mt) * chunk * 2, sums = (size_t)strips * mt * 1024;
    return waves * (staging > sums ? staging : sums);
}

template <int MT, int NS, int CK, int DEPTH, typename TO, bool SW, bool TL>
static void skinny_launch_kernel(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                                 int waves, hipStream_t stream) {
    const size_t smem = skinny_lds(MT, NS, CK, waves);
    const dim3 grid(ceil_div(N, 16 * NS)), block(waves * 64);
    if (smem > 64 * 1024)                            // beyond the default limit of dynamic LDS
        (void)hipFuncSetAttribute((const void*)linear_skinny_kernel<MT, NS, CK, DEPTH, TO, SW, TL>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL((linear_skinny_kernel<MT, NS, CK, DEPTH, TO, SW, TL>), grid, block, smem, stream,
                       (const bf16*)x, (const bf16*)w, bias, (TO*)out, M, N, K);
}

template <int MT, int NS, int CK, int DEPTH, typename TO>
static int skinny_launch(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int waves,
                         bool swiglu, hipStream_t stream) {
    const bool tail = K % CK != 0;
    if constexpr (NS >= 2) {
        if (swiglu) {
            if (tail) skinny_launch_kernel<MT, NS, CK, DEPTH, TO, true, true>(x, w, bias, out, M, N, K, waves, stream);
            else skinny_launch_kernel<MT, NS, CK, DEPTH, TO, true, false>(x, w, bias, out, M, N, K, waves, stream);
            SOMI_LAUNCH_CHECK("linear_skinny");
            return 0;
        }
    }
    if (tail) skinny_launch_kernel<MT, NS, CK, DEPTH, TO, false, true>(x, w, bias, out, M, N, K, waves, stream);
    else skinny_launch_kernel<MT, NS, CK, DEPTH, TO, false, false>(x, w, bias, out, M, N, K, waves, stream);
    SOMI_LAUNCH_CHECK("linear_skinny");
    return 0;
}

// The shapes that are built: 1, 2 or 4 strips with chunks of 64, two chunks in flight.
template <int MT, typename TO>
static int skinny_strips(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int waves,
                         int strips, bool swiglu, hipStream_t stream) {
    if (strips >= 4) return skinny_launch<MT, 4, 64, 2, TO>(x, w, bias, out, M, N, K, waves, swiglu, stream);
    if (strips >= 2) return skinny_launch<MT, 2, 64, 2, TO>(x, w, bias, out, M, N, K, waves, swiglu, stream);
    return skinny_launch<MT, 1, 64, 2, TO>(x, w, bias, out, M, N, K, waves, swiglu, stream);
}

static int skinny_dispatch(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M, int N,
                           int K, int waves, int strips, bool swiglu, hipStream_t stream) {
    const int mt = ceil_div(M, 16);
    SOMI_REQUIRE(skinny_lds(mt, strips, 64, waves) <= 160 * 1024,
                 "linear_skinny: %d wavefronts with %d strips need more than 160 KB of LDS", waves, strips);
#define SOMI_SKINNY(MT)                                                                                              \
    return out_dtype == SOMI_BF16 ? skinny_strips<MT, bf16>(x, w, bias, out, M, N, K, waves, strips, swiglu, stream)  \
                                  : skinny_strips<MT, float>(x, w, bias, out, M, N, K, waves, strips, swiglu, stream)
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
    SOMI_REQUIRE((int64_t)K * 2 * 64 < (int64_t)1 << 31, "linear_skinny: K (%d) is too large", K);
    SOMI_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "linear_skinny: x and w must be 16-byte aligned");
    SOMI_REQUIRE(out_dtype == SOMI_BF16 || out_dtype == SOMI_F32, "linear_skinny: unknown out dtype %d", out_dtype);
    return 0;
}

static int skinny_auto(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M, int N, int K,
                       bool swiglu, hipStream_t stream) {
    // Launch shape, from measurements at 7B layer sizes on MI355X.  8 wavefronts split K.  A workgroup
    // takes 2 (or 4) strips, reading x once for all of them, where that still leaves a workgroup for
    // most compute units and x is more than a few rows; one strip otherwise.
    const int mt = ceil_div(M, 16);
    const int blocks16 = ceil_div(N, 16);
    int strips = 1;
    if (blocks16 >= 256) strips = 2;
    if (blocks16 >= 2048 && M <= 4) strips = 1;
    if (blocks16 >= 4096 && mt >= 2) strips = 4;
    if (swiglu && strips < 2) strips = 2;
    int waves = SKINNY_MAX_WAVES;
    while (waves > 1 && waves * 64 > K + 63) waves /= 2;           // no more wavefronts than chunks of K
    return skinny_dispatch(x, w, bias, out, out_dtype, M, N, K, waves, strips, swiglu, stream);
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

// The same product with the launch shape given by the caller (wavefronts per workgroup: 1 to 8; 16-column
// strips per workgroup: 1, 2 or 4): for measuring how the shape should be chosen.
extern "C" int somi_linear_skinny_shaped(const void* x, const void* w, const float* bias, void* out, int out_dtype,
                                         int M, int N, int K, int waves, int strips, hipStream_t stream) {
    if (skinny_check(x, w, out_dtype, M, N, K)) return 1;
    SOMI_REQUIRE(strips == 1 || strips == 2 || strips == 4, "linear_skinny: strips must be 1, 2 or 4");
    SOMI_REQUIRE(waves >= 1 && waves <= SKINNY_MAX_WAVES, "linear_skinny: bad wavefront count %d", waves);
    if (M == 0) return 0;
    return skinny_dispatch(x, w, bias, out, out_dtype, M, N, K, waves, strips, false, stream);
}
