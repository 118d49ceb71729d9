// Linear layer for some tens of rows (decode batches of 17 to 64 requests): out[m, n] = sum_k x[m, k] * w[n, k]
// (+ bias[n]), bfloat16 in, float32 accumulation on the matrix cores.
//
// Reference: the same nn.Linear products as linear_plain.hip (somi_inference/models/qwen2.py:221-222,
// 268-271); the reference leaves them to a library.  The product is still bound by reading w once, but
// with this many rows x is no longer small: where every wavefront fetches its own pieces of x (as
// linear_skinny.hip does) the traffic of x from L2 is a multiple of the weight stream.  Here
//   * a workgroup of 4 wavefronts owns 64 * NS output columns and all rows of x; a wavefront owns
//     16 * NS of the columns, so no sums cross wavefronts;
//   * the wavefronts walk K together in chunks of 64: the chunk of x is loaded once by the whole
//     workgroup into (double-buffered, swizzled) LDS and read by all four; each wavefront turns its own
//     rows of w through a private piece of LDS into the operand layout, as in linear_skinny.hip;
//   * two chunks are in flight in registers; loads are buffer loads whose range ends at the last valid
//     row, so rows past N or M and a chunk that crosses K read as zero without a branch;
//   * K is also split over blockIdx.y where the columns alone do not fill the device.  Each split writes
//     its partial sums to a workspace and a second, small kernel adds them in split order (a fixed
//     order of additions) and applies the epilogue.  (Letting the last workgroup of a tile do that
//     behind device-scope fences was measured 4 times slower: on this part such a fence writes back
//     and invalidates a whole L2.)
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

#define SOMI_BUFFER_WORD3 0x00020000u            // raw buffer, 32-bit elements, no swizzle
#define SOMI_OUT_OF_RANGE 0x80000000u
#define MID_WAVES 4

// D[row = (lane / 16) * 4 + i][col = lane % 16]: a lane holds four consecutive output columns of row
// (lane % 16) of each 16-row tile of x, for each of its wavefront's strips.
template <int MT, int NS, typename TO, bool SWIGLU>
__device__ __forceinline__ void mid_epilogue(const f32x4 (&acc)[NS][MT], const float* __restrict__ bias,
                                             TO* __restrict__ out, int M, int N, int n0, int wave, int lane) {
    const int r = lane & 15, g = lane >> 4;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        if (m >= M) continue;
        if (SWIGLU) {
            // w holds gate and up rows interleaved in blocks of 16: strips 2p and 2p + 1 of a wavefront are
            // gate and up of the same 16 output columns
            const int n_out = N / 2;
#pragma unroll
            for (int p = 0; p < NS / 2; ++p) {
                const int n = (n0 + (wave * NS + 2 * p) * 16) / 2 + g * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float gate = acc[2 * p][mt][i], up = acc[2 * p + 1][mt][i];
                    if (n + i < n_out) out[(int64_t)m * n_out + n + i] = from_float<TO>(gate / (1.0f + expf(-gate)) * up);
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const int n = n0 + (wave * NS + s) * 16 + g * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) out[(int64_t)m * N + n + i] = from_float<TO>(acc[s][mt][i] + (bias ? bias[n + i] : 0.f));
            }
        }
    }
}

template <int MT, int NS, int CK, int DEPTH, typename TO, bool SWIGLU, bool TAIL>
__global__ void __launch_bounds__(MID_WAVES * 64, 2)
linear_mid_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias,
                  TO* __restrict__ out, int M, int N, int K, int chunks_per_split, float* __restrict__ partial) {
    constexpr int ROW_BYTES = CK * 2;              // bytes of a row in a chunk: 128 or 256
    constexpr int LPR = ROW_BYTES / 16;            // lanes that read one row: 8 or 16
    constexpr int WRPI = 64 / LPR;                 // rows a wavefront fetches with one load: 8 or 4
    constexpr int XRPI = 256 / LPR;                // rows the workgroup fetches with one load: 32 or 16
    constexpr int WLD = NS * 16 / WRPI;            // loads of w per thread and chunk
    constexpr int XL = (MT * 16 + XRPI - 1) / XRPI;   // loads of x per thread and chunk
    constexpr int X_BYTES = MT * 16 * ROW_BYTES, W_BYTES = NS * 16 * ROW_BYTES;
    __shared__ __attribute__((aligned(16))) char xs[2][X_BYTES];
    __shared__ __attribute__((aligned(16))) char ws[MID_WAVES][W_BYTES];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    const int tile = blockIdx.x, split = blockIdx.y, splits = gridDim.y;
    const int n0 = tile * (64 * NS);

    const int rows_here = min(64 * NS, N - n0);
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(w + (int64_t)n0 * K), 0, (int)((int64_t)rows_here * K * 2), SOMI_BUFFER_WORD3);
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(
        (void*)x, 0, (int)((int64_t)M * K * 2), SOMI_BUFFER_WORD3);

    // w: LPR lanes of a wavefront read one row's bytes of the chunk, 16 each; x: the same with all 256
    // threads.  Both land in LDS rows whose 16-byte pieces are XOR-swizzled with bits of the row number, so
    // that neither these row-wise writes nor the column-wise operand reads collide.
    const int lchunk = lane % LPR;
    auto swizzle = [](int row16) { return CK == 128 ? (row16 & 15) : ((row16 & 7) ^ (row16 >> 3)); };
    unsigned wgoff[WLD];
    int wsoff[WLD];
#pragma unroll
    for (int i = 0; i < WLD; ++i) {
        const int row = i * WRPI + lane / LPR;     // row among the wavefront's NS * 16
        wgoff[i] = ((unsigned)(wave * NS * 16 + row) * (unsigned)K + lchunk * 8) * 2u;
        wsoff[i] = row * ROW_BYTES + ((lchunk ^ swizzle(row & 15)) << 4);
    }
    unsigned xgoff[XL];
    int xsoff[XL];
    bool xkeep[XL];
#pragma unroll
    for (int j = 0; j < XL; ++j) {
        const int row = j * XRPI + tid / LPR;
        xgoff[j] = ((unsigned)row * (unsigned)K + lchunk * 8) * 2u;
        xsoff[j] = row * ROW_BYTES + ((lchunk ^ swizzle(row & 15)) << 4);
        xkeep[j] = row < MT * 16;
    }
    const int rswz = swizzle(r);

    f32x4 acc[NS][MT];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int chunks = (K + CK - 1) / CK;
    const int first = split * chunks_per_split;
    const int count = max(0, min(chunks_per_split, chunks - first));       // the same for every wavefront

    struct Stage {
        u32x4 wv[WLD];
        u32x4 xv[XL];
    };
    auto issue = [&](Stage& st, int at) {
        const int k0 = (first + at) * CK;
        const bool inside = !TAIL || k0 + lchunk * 8 < K;
#pragma unroll
        for (int i = 0; i < WLD; ++i)
            st.wv[i] = __builtin_amdgcn_raw_buffer_load_b128(
                wres, inside ? wgoff[i] + (unsigned)k0 * 2u : SOMI_OUT_OF_RANGE, 0, 0);
#pragma unroll
        for (int j = 0; j < XL; ++j)
            st.xv[j] = __builtin_amdgcn_raw_buffer_load_b128(
                xres, inside ? xgoff[j] + (unsigned)k0 * 2u : SOMI_OUT_OF_RANGE, 0, 0);
    };
    auto stash = [&](const Stage& st, int buf) {
#pragma unroll
        for (int i = 0; i < WLD; ++i) *reinterpret_cast<u32x4*>(ws[wave] + wsoff[i]) = st.wv[i];
#pragma unroll
        for (int j = 0; j < XL; ++j)
            if (xkeep[j]) *reinterpret_cast<u32x4*>(xs[buf] + xsoff[j]) = st.xv[j];
    };
    // the k-values of a 64-wide block are dealt to the two products as 16-byte pieces 2g and 2g + 1 of lane
    // group g: any order serves as long as w and x use the same
    auto compute = [&](int buf) {
#pragma unroll
        for (int cb = 0; cb < CK / 64; ++cb) {
            bf16x8 xa[MT], xb[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const char* row = xs[buf] + (mt * 16 + r) * ROW_BYTES;
                xa[mt] = *reinterpret_cast<const bf16x8*>(row + (((cb * 8 + 2 * g) ^ rswz) << 4));
                xb[mt] = *reinterpret_cast<const bf16x8*>(row + (((cb * 8 + 2 * g + 1) ^ rswz) << 4));
            }
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const char* row = ws[wave] + (s * 16 + r) * ROW_BYTES;
                const bf16x8 wa = *reinterpret_cast<const bf16x8*>(row + (((cb * 8 + 2 * g) ^ rswz) << 4));
                const bf16x8 wb = *reinterpret_cast<const bf16x8*>(row + (((cb * 8 + 2 * g + 1) ^ rswz) << 4));
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xa[mt], acc[s][mt], 0, 0, 0);
                    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb, xb[mt], acc[s][mt], 0, 0, 0);
                }
            }
        }
    };
    // One barrier per chunk: chunk i goes to x buffer i % 2; a wavefront that writes buffer i % 2 has
    // passed the barrier of chunk i - 1, so every wavefront is done reading chunk i - 2 from it.
    // DEPTH chunks are in flight in registers: set d holds chunk `at + d`.  The loop is entered on one
    // path only, with every set issued, so that the waits inside it count loads exactly.
    Stage st[DEPTH];
    int done = 0;                                    // chunks computed so far: the x buffer of the next one is done % 2
    auto step = [&](Stage& stage, int refill) {
        stash(stage, done & 1);
        if (refill >= 0) issue(stage, refill);
        __syncthreads();
        compute(done & 1);
        ++done;
    };
    if (count >= DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) issue(st[d], d);
        int at = 0;
        for (; at + 2 * DEPTH - 1 < count; at += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) step(st[d], at + DEPTH + d);
        }
        // DEPTH to 2 * DEPTH - 1 chunks are left
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) step(st[d], (d < DEPTH - 1 && at + DEPTH + d < count) ? at + DEPTH + d : -1);
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (at + DEPTH + d < count) step(st[d], -1);
    } else {
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (d < count) issue(st[d], d);
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (d < count) step(st[d], -1);
    }

    if (splits > 1) {
        // partial sums in the accumulators' own layout: [split][tile][wave][strip][row tile][lane][4]
        float* mine = partial + ((int64_t)(split * gridDim.x + tile) * MID_WAVES + wave) * (NS * MT * 256) + lane * 4;
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) *reinterpret_cast<f32x4*>(mine + (s * MT + mt) * 256) = acc[s][mt];
        return;
    }
    mid_epilogue<MT, NS, TO, SWIGLU>(acc, bias, out, M, N, n0, wave, lane);
}

// Adds the partial sums of the splits in split order and applies the epilogue: one workgroup per column tile.
template <int MT, int NS, typename TO, bool SWIGLU>
__global__ void __launch_bounds__(MID_WAVES * 64)
linear_mid_reduce_kernel(const float* __restrict__ partial, const float* __restrict__ bias, TO* __restrict__ out,
                         int M, int N, int splits) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, tile = blockIdx.x;
    f32x4 acc[NS][MT];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int sp = 0; sp < splits; ++sp) {
        const float* theirs = partial + ((int64_t)(sp * gridDim.x + tile) * MID_WAVES + wave) * (NS * MT * 256) + lane * 4;
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[s][mt] += *reinterpret_cast<const f32x4*>(theirs + (s * MT + mt) * 256);
    }
    mid_epilogue<MT, NS, TO, SWIGLU>(acc, bias, out, M, N, tile * (64 * NS), wave, lane);
}

template <int MT, int NS, int CK, int DEPTH, typename TO, bool SW, bool TL>
static void mid_launch_kernel(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                              int splits, int chunks_per_split, float* partial, hipStream_t stream) {
    const dim3 grid(ceil_div(N, 64 * NS), splits), block(MID_WAVES * 64);
    hipLaunchKernelGGL((linear_mid_kernel<MT, NS, CK, DEPTH, TO, SW, TL>), grid, block, 0, stream, (const bf16*)x,
                       (const bf16*)w, bias, (TO*)out, M, N, K, chunks_per_split, partial);
    if (splits > 1)
        hipLaunchKernelGGL((linear_mid_reduce_kernel<MT, NS, TO, SW>), dim3(grid.x), block, 0, stream,
                           (const float*)partial, bias, (TO*)out, M, N, splits);
}

template <int MT, int NS, int CK, int DEPTH, typename TO>
static int mid_launch(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int splits,
                      bool swiglu, float* partial, hipStream_t stream) {
    const bool tail = K % CK != 0;
    const int chunks_per_split = ceil_div(ceil_div(K, CK), splits);
    if constexpr (NS >= 2) {
        if (swiglu) {
            if (tail) mid_launch_kernel<MT, NS, CK, DEPTH, TO, true, true>(x, w, bias, out, M, N, K, splits, chunks_per_split, partial, stream);
            else mid_launch_kernel<MT, NS, CK, DEPTH, TO, true, false>(x, w, bias, out, M, N, K, splits, chunks_per_split, partial, stream);
            SOMI_LAUNCH_CHECK("linear_mid");
            return 0;
        }
    }
    if (tail) mid_launch_kernel<MT, NS, CK, DEPTH, TO, false, true>(x, w, bias, out, M, N, K, splits, chunks_per_split, partial, stream);
    else mid_launch_kernel<MT, NS, CK, DEPTH, TO, false, false>(x, w, bias, out, M, N, K, splits, chunks_per_split, partial, stream);
    SOMI_LAUNCH_CHECK("linear_mid");
    return 0;
}

// A program that measures other shapes (chunk sizes, depths) can include this file with SOMI_MID_NO_ENTRY_POINTS
// defined and instantiate the launchers above itself; the library builds what follows.
#ifndef SOMI_MID_NO_ENTRY_POINTS
#define MID_CK 64                                // K values per chunk and chunks in flight of the shapes that are built
#define MID_DEPTH 2

template <int MT, typename TO>
static int mid_strips(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int strips,
                      int splits, bool swiglu, float* partial, hipStream_t stream) {
    if (strips >= 2) return mid_launch<MT, 2, MID_CK, MID_DEPTH, TO>(x, w, bias, out, M, N, K, splits, swiglu, partial, stream);
    return mid_launch<MT, 1, MID_CK, MID_DEPTH, TO>(x, w, bias, out, M, N, K, splits, swiglu, partial, stream);
}

// Floats of workspace one launch needs: the partial sums of every split (nothing for one split).
static int64_t mid_workspace_floats(int M, int N, int strips, int splits) {
    if (splits <= 1) return 0;
    const int mt = ceil_div(M, 16);
    return (int64_t)splits * ceil_div(N, 64 * strips) * MID_WAVES * strips * mt * 256;
}

// The launch shape: strips per wavefront and splits of K.  Two strips where the columns still give every
// compute unit a workgroup; K is split until there are about two workgroups per compute unit, in
// pieces of at least 8 chunks, within the workspace.  Chosen by whole decode steps of 64 requests at 7B
// layer sizes (7.7 ms with this rule: down in 8 splits, gate_up in 2; 8.0 ms with at most 5 or 3 splits,
// 7.9 ms with twice as many); timing the kernel alone in a loop ranks the shapes differently.
static void mid_shape(int M, int N, int K, bool swiglu, int64_t workspace_floats, int* strips, int* splits) {
    const int chunks = ceil_div(K, MID_CK);
    int ns = (swiglu || ceil_div(N, 128) >= 256) ? 2 : 1;
    int tiles = ceil_div(N, 64 * ns);
    int ks = 1;
    if (tiles < 384) {
        ks = min(ceil_div(448, tiles), max(1, chunks / 8));
        const int per = ceil_div(chunks, ks);
        ks = ceil_div(chunks, per);                  // no empty split
    }
    while (ks > 1 && mid_workspace_floats(M, N, ns, ks) > workspace_floats) --ks;
    if (ks > 1) ks = ceil_div(chunks, ceil_div(chunks, ks));
    *strips = ns;
    *splits = ks;
}

static int mid_check(const void* x, const void* w, int out_dtype, int M, int N, int K) {
    SOMI_REQUIRE(M >= 0 && N > 0 && K > 0, "linear_mid: bad sizes M=%d N=%d K=%d", M, N, K);
    SOMI_REQUIRE(M <= 64, "linear_mid: at most 64 rows, got %d", M);
    SOMI_REQUIRE(K % 8 == 0, "linear_mid: K (%d) must be a multiple of 8", K);
    SOMI_REQUIRE((int64_t)K * 2 * 128 < (int64_t)1 << 31, "linear_mid: K (%d) is too large", K);
    SOMI_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "linear_mid: x and w must be 16-byte aligned");
    SOMI_REQUIRE(out_dtype == SOMI_BF16 || out_dtype == SOMI_F32, "linear_mid: unknown out dtype %d", out_dtype);
    return 0;
}

static int mid_dispatch(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M, int N, int K,
                        int strips, int splits, bool swiglu, float* partial, hipStream_t stream) {
    const int mt = ceil_div(M, 16);
#define SOMI_MID(MT)                                                                                                 \
    return out_dtype == SOMI_BF16                                                                                    \
               ? mid_strips<MT, bf16>(x, w, bias, out, M, N, K, strips, splits, swiglu, partial, stream) \
               : mid_strips<MT, float>(x, w, bias, out, M, N, K, strips, splits, swiglu, partial, stream)
    switch (mt) {
        case 1: SOMI_MID(1);
        case 2: SOMI_MID(2);
        case 3: SOMI_MID(3);
        default: SOMI_MID(4);
    }
#undef SOMI_MID
}

// x: [M, K] bfloat16, w: [N, K] bfloat16, bias: [N] float32 or null, out: [M, N] bfloat16 or float32 (with
// swiglu: w is [2 I, K] with gate and up rows interleaved in blocks of 16, no bias, out: [M, I]).  M <= 64;
// K a multiple of 8.  workspace: `workspace_floats` floats for the partial sums of a split K (may be null:
// then K is not split).  Launches that share a workspace must not overlap (one stream).
extern "C" int somi_linear_mid(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M, int N,
                               int K, int swiglu, float* workspace, int64_t workspace_floats, hipStream_t stream) {
    if (mid_check(x, w, out_dtype, M, N, K)) return 1;
    SOMI_REQUIRE(!swiglu || (N % 32 == 0 && bias == nullptr), "linear_mid: the gated form needs whole pairs of strips and no bias");
    if (M == 0) return 0;
    int strips, splits;
    mid_shape(M, N, K, swiglu != 0, workspace ? workspace_floats : 0, &strips, &splits);
    return mid_dispatch(x, w, bias, out, out_dtype, M, N, K, strips, splits, swiglu != 0, workspace, stream);
}

// The same product with the launch shape given by the caller: for measuring how the shape should be chosen.
extern "C" int somi_linear_mid_shaped(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M,
                                      int N, int K, int swiglu, int strips, int splits, float* workspace,
                                      int64_t workspace_floats, hipStream_t stream) {
    if (mid_check(x, w, out_dtype, M, N, K)) return 1;
    SOMI_REQUIRE(strips == 1 || strips == 2, "linear_mid: strips must be 1 or 2");
    SOMI_REQUIRE(!swiglu || (strips == 2 && N % 32 == 0 && bias == nullptr), "linear_mid: the gated form needs pairs of strips and no bias");
    SOMI_REQUIRE(splits >= 1 && splits <= ceil_div(K, MID_CK), "linear_mid: bad number of splits %d", splits);
    SOMI_REQUIRE(splits == 1 || (workspace && mid_workspace_floats(M, N, strips, splits) <= workspace_floats),
                 "linear_mid: %d splits need %lld floats of workspace", splits,
                 (long long)mid_workspace_floats(M, N, strips, splits));
    if (M == 0) return 0;
    return mid_dispatch(x, w, bias, out, out_dtype, M, N, K, strips, splits, swiglu != 0, workspace, stream);
}
#endif
