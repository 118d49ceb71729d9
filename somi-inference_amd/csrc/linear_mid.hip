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
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

#define SOMI_BUFFER_WORD3 0x00020000u            // raw buffer, 32-bit elements, no swizzle
#define SOMI_OUT_OF_RANGE 0x80000000u
#define MID_WAVES 4

#define MID_PLAIN 0
#define MID_SCALED 1        // out = s[m] * (x . w^T) (+ bias): the product of RMS-normed rows, see linear_fused.hip
#define MID_RESIDUAL 2      // h += x . w^T (+ bias) in float32, with the next norm's rows and the rows' sums of squares

// What the fused forms need beside the product's own arguments (see linear_fused.hip for the arithmetic).
struct MidFusion {
    float* h;                 // residual: [M, N] float32, in and out
    const float* norm_w;      // residual: the next norm's weight [N], or null
    bf16* xnext;              // residual: [M, N] = bfloat16(norm_w * h), or null
    float* stats_out;         // residual: [column tiles][16 MT] sums of squares of the new h over the tile's columns
    int stats_stride;         // floats from one row of either table to the next, or 0 for 16 MT
    const float* stats_in;    // scaled: [stats_blocks][16 MT] partial sums of squares of the rows that were normed
    int stats_blocks;
    float eps;
};

// What the end of a fused product reads beside the sums, fetched ahead of its use (in the kernel that adds the
// splits: before the partial sums, so that the latencies overlap).  MTH: the 16-row tiles the caller holds.
#define MID_STATS_AHEAD 16
template <int MTH, int NS, int FUSE>
struct MidAhead {
    float stats[FUSE == MID_SCALED ? MID_STATS_AHEAD : 1][MTH];
    f32x4 h[FUSE == MID_RESIDUAL ? NS : 1][FUSE == MID_RESIDUAL ? MTH : 1];
};

// The producer's partial sums of squares [stats_blocks][rows_total] are added in a fixed order: lane l of
// wavefront v adds the rows first_row + MTH (l % 16) .. + MTH - 1 of the workgroups 4 v + l / 16, that + 16, ...;
// then a thread per row adds those 16 sums in order.  MTH consecutive floats are one load.
template <int MTH>
__device__ __forceinline__ void mid_stats_load(float (&to)[MTH], const float* __restrict__ stats, int block, int blocks,
                                               int rows_total, int first_row) {
    const float* from = stats + (int64_t)block * rows_total + first_row + (threadIdx.x & 15) * MTH;
    if (block < blocks) {
        __builtin_memcpy(&to[0], __builtin_assume_aligned(from, MTH == 3 ? 4 : 4 * MTH), 4 * MTH);
    } else {
#pragma unroll
        for (int j = 0; j < MTH; ++j) to[j] = 0.f;
    }
}

// Four consecutive elements of a row are one access where the row length and the addresses keep them aligned
// and inside together.
__device__ __forceinline__ bool mid_whole(int N, const float* bias, const MidFusion& fusion) {
    return (N & 3) == 0 && (((uintptr_t)bias | (uintptr_t)fusion.h | (uintptr_t)fusion.norm_w) & 15) == 0 &&
           ((uintptr_t)fusion.xnext & 7) == 0;
}

__device__ __forceinline__ f32x4 mid_load4(const float* __restrict__ from, int n, int N, bool whole) {
    if (whole) return *reinterpret_cast<const f32x4*>(from);
    f32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = n + i < N ? from[i] : 0.f;
    return v;
}

template <int MTH, int NS, int FUSE>
__device__ __forceinline__ void mid_fetch_ahead(MidAhead<MTH, NS, FUSE>& ahead, const MidFusion& fusion, int M, int N,
                                                const float* bias, int n0, int rows_total, int first_row) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    if constexpr (FUSE == MID_SCALED) {
#pragma unroll
        for (int i = 0; i < MID_STATS_AHEAD; ++i)
            mid_stats_load<MTH>(ahead.stats[i], fusion.stats_in, wave * 4 + g + i * 16, fusion.stats_blocks, rows_total,
                                first_row);
    }
    if constexpr (FUSE == MID_RESIDUAL) {
        const bool whole = mid_whole(N, bias, fusion);
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int mt = 0; mt < MTH; ++mt) {
                const int m = first_row + mt * 16 + r, n = n0 + (wave * NS + s) * 16 + g * 4;
                ahead.h[s][mt] = m < M && n < N ? mid_load4(fusion.h + (int64_t)m * N + n, n, N, whole)
                                                : f32x4{0.f, 0.f, 0.f, 0.f};
            }
    }
}

// The end of a product: bias / gate / fused forms on the sums a lane holds for the MTH 16-row tiles from row
// first_row on (rows_total = 16 ceil(M / 16) is the width of the row statistics).
// D[row = (lane / 16) * 4 + i][col = lane % 16]: a lane holds four consecutive output columns of row
// (lane % 16) of each 16-row tile of x, for each of its wavefront's strips.
template <int MTH, int NS, typename TO, bool SWIGLU, int FUSE>
__device__ __forceinline__ void mid_finish(f32x4 (&acc)[NS][MTH], const MidAhead<MTH, NS, FUSE>& ahead,
                                           const float* __restrict__ bias, TO* __restrict__ out,
                                           const MidFusion& fusion, int M, int N, int K, int n0, int tile,
                                           int rows_total, int first_row) {
    constexpr int ROWS = 16 * MTH;
    __shared__ float shared_sums[16 * 64];         // [wave][lane group][row]
    __shared__ float row_scale[64];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    if constexpr (FUSE == MID_SCALED) {
        float mine[MTH];
#pragma unroll
        for (int j = 0; j < MTH; ++j) mine[j] = 0.f;
#pragma unroll
        for (int i = 0; i < MID_STATS_AHEAD; ++i)
#pragma unroll
            for (int j = 0; j < MTH; ++j) mine[j] += ahead.stats[i][j];
        for (int b = wave * 4 + g + MID_STATS_AHEAD * 16; b < fusion.stats_blocks; b += 16) {
            float more[MTH];
            mid_stats_load<MTH>(more, fusion.stats_in, b, fusion.stats_blocks, rows_total, first_row);
#pragma unroll
            for (int j = 0; j < MTH; ++j) mine[j] += more[j];
        }
#pragma unroll
        for (int j = 0; j < MTH; ++j) shared_sums[(wave * 4 + g) * ROWS + r * MTH + j] = mine[j];
        __syncthreads();
        if (tid < ROWS) {
            float sum = 0.f;
#pragma unroll
            for (int group = 0; group < 16; ++group) sum += shared_sums[group * ROWS + tid];
            row_scale[tid] = 1.0f / sqrtf(sum / (float)K + fusion.eps);
        }
        __syncthreads();
    }
    if constexpr (SWIGLU) {
        // w holds gate and up rows interleaved in blocks of 16: strips 2p and 2p + 1 of a wavefront are
        // gate and up of the same 16 output columns
        const int n_out = N / 2;
#pragma unroll
        for (int mt = 0; mt < MTH; ++mt) {
            const int m = first_row + mt * 16 + r;
            if (m >= M) continue;
            float scale = 1.0f;
            if constexpr (FUSE == MID_SCALED) scale = row_scale[mt * 16 + r];
#pragma unroll
            for (int p = 0; p < NS / 2; ++p) {
                const int n = (n0 + (wave * NS + 2 * p) * 16) / 2 + g * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float gate = acc[2 * p][mt][i] * scale, up = acc[2 * p + 1][mt][i] * scale;
                    if (n + i < n_out) out[(int64_t)m * n_out + n + i] = from_float<TO>(gate / (1.0f + expf(-gate)) * up);
                }
            }
        }
        return;
    }
    const bool whole = mid_whole(N, bias, fusion);
    float squares[MTH];
#pragma unroll
    for (int mt = 0; mt < MTH; ++mt) squares[mt] = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int n = n0 + (wave * NS + s) * 16 + g * 4;
        if (n >= N) continue;
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        const f32x4 bias4 = bias ? mid_load4(bias + n, n, N, whole) : zero;
        f32x4 norm4 = zero;
        if constexpr (FUSE == MID_RESIDUAL)
            if (fusion.xnext) norm4 = mid_load4(fusion.norm_w + n, n, N, whole);
#pragma unroll
        for (int mt = 0; mt < MTH; ++mt) {
            const int m = first_row + mt * 16 + r;
            if (m >= M) continue;
            const int64_t at = (int64_t)m * N + n;
            if constexpr (FUSE == MID_RESIDUAL) {
                const f32x4 now = ahead.h[s][mt] + acc[s][mt] + bias4;
                if (whole) {
                    *reinterpret_cast<f32x4*>(fusion.h + at) = now;
                    if (fusion.xnext) {
                        bf16x4 next;
#pragma unroll
                        for (int i = 0; i < 4; ++i) next[i] = (bf16)(norm4[i] * now[i]);
                        *reinterpret_cast<bf16x4*>(fusion.xnext + at) = next;
                    }
                    squares[mt] += now[0] * now[0] + now[1] * now[1] + now[2] * now[2] + now[3] * now[3];
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (n + i >= N) continue;
                        fusion.h[at + i] = now[i];
                        if (fusion.xnext) fusion.xnext[at + i] = (bf16)(norm4[i] * now[i]);
                        squares[mt] += now[i] * now[i];
                    }
                }
            } else {
                float scale = 1.0f;
                if constexpr (FUSE == MID_SCALED) scale = row_scale[mt * 16 + r];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) out[at + i] = from_float<TO>(acc[s][mt][i] * scale + bias4[i]);
            }
        }
    }
    if constexpr (FUSE == MID_RESIDUAL) {
        // a row's squares over the tile's columns: the four lane groups of the four wavefronts, in that order
#pragma unroll
        for (int mt = 0; mt < MTH; ++mt) shared_sums[(wave * 4 + g) * 64 + mt * 16 + r] = squares[mt];
        __syncthreads();
        if (tid < ROWS) {
            float total = 0.f;
#pragma unroll
            for (int part = 0; part < 16; ++part) total += shared_sums[part * 64 + tid];
            fusion.stats_out[(int64_t)tile * rows_total + first_row + tid] = total;
        }
    }
}

template <int MT, int NS, int CK, int DEPTH, typename TO, bool SWIGLU, bool TAIL, int FUSE>
__global__ void __launch_bounds__(MID_WAVES * 64, 2)
linear_mid_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w, const float* __restrict__ bias,
                  TO* __restrict__ out, int M, int N, int K, int chunks_per_split, float* __restrict__ partial,
                  MidFusion fusion) {
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
                wres, inside ? wgoff[i] + (unsigned)k0 * 2u : SOMI_OUT_OF_RANGE, 0, SOMI_LOAD_ONCE);
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
    MidAhead<MT, NS, FUSE> ahead;
    const int stats_stride = fusion.stats_stride > 0 ? fusion.stats_stride : 16 * MT;
    mid_fetch_ahead(ahead, fusion, M, N, bias, n0, stats_stride, 0);
    mid_finish<MT, NS, TO, SWIGLU, FUSE>(acc, ahead, bias, out, fusion, M, N, K, n0, tile, stats_stride, 0);
}

// Adds the partial sums of the splits in split order and applies the epilogue: one workgroup per column tile
// and 16-row tile (blockIdx.y).
template <int MT, int NS, typename TO, bool SWIGLU, int FUSE>
__global__ void __launch_bounds__(MID_WAVES * 64)
linear_mid_reduce_kernel(const float* __restrict__ partial, const float* __restrict__ bias, TO* __restrict__ out,
                         int M, int N, int K, int splits, MidFusion fusion) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, tile = blockIdx.x, mt = blockIdx.y;
    MidAhead<1, NS, FUSE> ahead;
    const int stats_stride = fusion.stats_stride > 0 ? fusion.stats_stride : 16 * MT;
    mid_fetch_ahead(ahead, fusion, M, N, bias, tile * (64 * NS), stats_stride, 16 * mt);
    f32x4 acc[NS][1];
#pragma unroll
    for (int s = 0; s < NS; ++s) acc[s][0] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int sp = 0; sp < splits; ++sp) {
        const float* theirs = partial + ((int64_t)(sp * gridDim.x + tile) * MID_WAVES + wave) * (NS * MT * 256) + lane * 4;
#pragma unroll
        for (int s = 0; s < NS; ++s) acc[s][0] += *reinterpret_cast<const f32x4*>(theirs + (s * MT + mt) * 256);
    }
    mid_finish<1, NS, TO, SWIGLU, FUSE>(acc, ahead, bias, out, fusion, M, N, K, tile * (64 * NS), tile, stats_stride, 16 * mt);
}

template <int MT, int NS, int CK, int DEPTH, typename TO, bool SW, bool TL, int FUSE>
static void mid_launch_kernel(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                              int splits, int chunks_per_split, float* partial, const MidFusion& fusion,
                              hipStream_t stream) {
    const dim3 grid(ceil_div(N, 64 * NS), splits), block(MID_WAVES * 64);
    hipLaunchKernelGGL((linear_mid_kernel<MT, NS, CK, DEPTH, TO, SW, TL, FUSE>), grid, block, 0, stream, (const bf16*)x,
                       (const bf16*)w, bias, (TO*)out, M, N, K, chunks_per_split, partial, fusion);
    if (splits > 1)
        hipLaunchKernelGGL((linear_mid_reduce_kernel<MT, NS, TO, SW, FUSE>), dim3(grid.x, MT), block, 0, stream,
                           (const float*)partial, bias, (TO*)out, M, N, K, splits, fusion);
}

template <int MT, int NS, int CK, int DEPTH, typename TO, int FUSE>
static int mid_launch(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int splits,
                      bool swiglu, float* partial, const MidFusion& fusion, hipStream_t stream) {
    const bool tail = K % CK != 0;
    const int chunks_per_split = ceil_div(ceil_div(K, CK), splits);
    if constexpr (NS >= 2 && FUSE != MID_RESIDUAL) {
        if (swiglu) {
            if (tail) mid_launch_kernel<MT, NS, CK, DEPTH, TO, true, true, FUSE>(x, w, bias, out, M, N, K, splits, chunks_per_split, partial, fusion, stream);
            else mid_launch_kernel<MT, NS, CK, DEPTH, TO, true, false, FUSE>(x, w, bias, out, M, N, K, splits, chunks_per_split, partial, fusion, stream);
            SOMI_LAUNCH_CHECK("linear_mid");
            return 0;
        }
    }
    if (tail) mid_launch_kernel<MT, NS, CK, DEPTH, TO, false, true, FUSE>(x, w, bias, out, M, N, K, splits, chunks_per_split, partial, fusion, stream);
    else mid_launch_kernel<MT, NS, CK, DEPTH, TO, false, false, FUSE>(x, w, bias, out, M, N, K, splits, chunks_per_split, partial, fusion, stream);
    SOMI_LAUNCH_CHECK("linear_mid");
    return 0;
}

#define MID_CK 64                                // K values per chunk and chunks in flight of the shapes that are built
#define MID_DEPTH 2

template <int MT, typename TO, int FUSE>
static int mid_strips(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int strips,
                      int splits, bool swiglu, float* partial, const MidFusion& fusion, hipStream_t stream) {
    if (strips >= 2) return mid_launch<MT, 2, MID_CK, MID_DEPTH, TO, FUSE>(x, w, bias, out, M, N, K, splits, swiglu, partial, fusion, stream);
    return mid_launch<MT, 1, MID_CK, MID_DEPTH, TO, FUSE>(x, w, bias, out, M, N, K, splits, swiglu, partial, fusion, stream);
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
// 7.9 ms with twice as many); timing the kernel alone in a loop ranks the shapes differently.  The counts go
// with the device's compute units (on the 256 of an MI355X: 448 workgroups aimed at, K split below 384 tiles, two
// strips from 256 tiles of 128 columns on).
#define MID_MIN_CHUNKS 8                      // chunks of K a split holds at least
static void mid_shape(int M, int N, int K, bool swiglu, int64_t workspace_floats, int units, int* strips, int* splits) {
    const int chunks = ceil_div(K, MID_CK);
    const int target = 7 * units / 4;         // K is split until about this many workgroups run
    int ns = (swiglu || ceil_div(N, 128) >= units) ? 2 : 1;
    int tiles = ceil_div(N, 64 * ns);
    int ks = 1;
    if (tiles < 3 * units / 2) {
        ks = min(ceil_div(target, tiles), max(1, chunks / MID_MIN_CHUNKS));
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

template <int FUSE>
static int mid_dispatch(const void* x, const void* w, const float* bias, void* out, int out_dtype, int M, int N, int K,
                        int strips, int splits, bool swiglu, float* partial, const MidFusion& fusion,
                        hipStream_t stream) {
    const int mt = ceil_div(M, 16);
#define SOMI_MID(MT)                                                                                                 \
    if constexpr (FUSE == MID_PLAIN) {                                                                               \
        if (out_dtype == SOMI_F32)                                                                                   \
            return mid_strips<MT, float, FUSE>(x, w, bias, out, M, N, K, strips, splits, swiglu, partial, fusion, stream); \
    }                                                                                                                \
    return mid_strips<MT, bf16, FUSE>(x, w, bias, out, M, N, K, strips, splits, swiglu, partial, fusion, stream)
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
    mid_shape(M, N, K, swiglu != 0, workspace ? workspace_floats : 0, somi_units(), &strips, &splits);
    return mid_dispatch<MID_PLAIN>(x, w, bias, out, out_dtype, M, N, K, strips, splits, swiglu != 0, workspace, MidFusion{}, stream);
}

// Column tiles (= rows of the statistics) that somi_linear_mid_residual launches for these sizes.
extern "C" int somi_linear_mid_residual_tiles(int M, int N, int K) {
    int strips, splits;
    mid_shape(M, N, K, false, 0, somi_units(), &strips, &splits);
    return ceil_div(N, 64 * strips);
}

// The product into the residual stream, as somi_linear_residual (linear_fused.hip) for up to 64 rows:
// h[m, n] += x[m, :] . w[n, :] (+ bias[n]) in float32; stats: [somi_linear_mid_residual_tiles()][16 ceil(M / 16)]
// float32 sums of squares of the new h per column tile and row (stats_stride: floats from one tile's sums to the
// next where they are columns of the table of more rows, a multiple of 4, or 0); xnext: [M, N] = bfloat16(norm_w * h),
// or null.
extern "C" int somi_linear_mid_residual(const void* x, const void* w, const float* bias, float* h, float* stats,
                                        int stats_stride, const float* norm_w, void* xnext, int M, int N, int K,
                                        float* workspace, int64_t workspace_floats, hipStream_t stream) {
    if (mid_check(x, w, SOMI_BF16, M, N, K)) return 1;
    SOMI_REQUIRE(h && stats, "linear_mid_residual: h and stats are needed");
    SOMI_REQUIRE(!xnext || norm_w, "linear_mid_residual: the next rows need the norm's weight");
    SOMI_REQUIRE(stats_stride == 0 || (stats_stride % 4 == 0 && stats_stride >= 16 * ceil_div(M, 16)),
                 "linear_mid_residual: a stride of %d floats does not hold the sums of %d rows", stats_stride, M);
    if (M == 0) return 0;
    int strips, splits;
    mid_shape(M, N, K, false, workspace ? workspace_floats : 0, somi_units(), &strips, &splits);
    MidFusion fusion{};
    fusion.h = h;
    fusion.norm_w = norm_w;
    fusion.xnext = (bf16*)xnext;
    fusion.stats_out = stats;
    fusion.stats_stride = stats_stride;
    return mid_dispatch<MID_RESIDUAL>(x, w, bias, nullptr, SOMI_BF16, M, N, K, strips, splits, false, workspace, fusion, stream);
}

// The product out of the residual stream, as somi_linear_scaled (linear_fused.hip) for up to 64 rows:
// out = s * (x . w^T) (+ bias), or the gated form on s g and s u, with s[m] = 1 / sqrt(sum of stats[:, m] / K + eps).
// stats: [stats_blocks][16 ceil(M / 16)] float32; out: bfloat16.
extern "C" int somi_linear_mid_scaled(const void* x, float eps, const float* stats, int stats_blocks, const void* w,
                                      const float* bias, void* out, int M, int N, int K, int swiglu, float* workspace,
                                      int64_t workspace_floats, hipStream_t stream) {
    if (mid_check(x, w, SOMI_BF16, M, N, K)) return 1;
    SOMI_REQUIRE(stats && stats_blocks > 0 && (uintptr_t)stats % 16 == 0, "linear_mid_scaled: the row statistics are needed, 16-byte aligned");
    SOMI_REQUIRE(!swiglu || (N % 32 == 0 && bias == nullptr), "linear_mid_scaled: the gated form needs whole pairs of strips and no bias");
    if (M == 0) return 0;
    int strips, splits;
    mid_shape(M, N, K, swiglu != 0, workspace ? workspace_floats : 0, somi_units(), &strips, &splits);
    MidFusion fusion{};
    fusion.stats_in = stats;
    fusion.stats_blocks = stats_blocks;
    fusion.eps = eps;
    return mid_dispatch<MID_SCALED>(x, w, bias, out, SOMI_BF16, M, N, K, strips, splits, swiglu != 0, workspace, fusion, stream);
}

// The plain product with the launch shape given by the caller: for measuring how the shape should be chosen.
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
    return mid_dispatch<MID_PLAIN>(x, w, bias, out, out_dtype, M, N, K, strips, splits, swiglu != 0, workspace, MidFusion{}, stream);
}

// The launch shape (strips per wavefront, splits of K) that the entry points above choose for these sizes on a device
// of `units` compute units (0: the current device): what a test of the choice asks without a GPU.
extern "C" int somi_linear_mid_choice(int M, int N, int K, int swiglu, int64_t workspace_floats, int units, int* strips,
                                      int* splits) {
    SOMI_REQUIRE(M > 0 && N > 0 && K > 0 && units >= 0 && strips && splits, "linear_mid_choice: bad arguments");
    mid_shape(M, N, K, swiglu != 0, workspace_floats, units > 0 ? units : somi_units(), strips, splits);
    return 0;
}
