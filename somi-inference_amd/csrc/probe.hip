// Two small measurements of the machine itself, for benchmarks that report a fraction of what it can do:
// how fast memory streams into the compute units, and how fast the matrix cores multiply bfloat16.
//
// Reference: the reference's benchmarks report times only (benchmarks/common.py:159-170); there is no
// counterpart.  Published peaks of an MI355X are 8 TB/s and 2.5 PFLOP/s (dense bfloat16); what a program can reach
// under the card's power limit is lower, and these kernels measure it.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

// Reads `pieces` 16-byte pieces once, every workgroup a contiguous share in steps of its NT lanes, DEPTH loads in
// flight a lane (NT: 256 or 512 lanes a workgroup; NONTEMPORAL: loads that tell the caches not to keep the line); the
// exclusive-or of everything read goes to out[blockIdx.x] so that no load can be dropped.
template <int NT, int DEPTH, bool NONTEMPORAL>
__global__ void __launch_bounds__(NT)
probe_stream_read_kernel(const u32x4* __restrict__ src, int64_t pieces, unsigned int* __restrict__ out) {
    const int64_t per_block = (pieces + gridDim.x - 1) / gridDim.x;
    const int64_t begin = per_block * blockIdx.x, end = begin + per_block < pieces ? begin + per_block : pieces;
    u32x4 acc = {0u, 0u, 0u, 0u};
    int64_t i = begin + threadIdx.x;
    for (; i + (DEPTH - 1) * NT < end; i += DEPTH * NT) {
        u32x4 v[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) v[d] = NONTEMPORAL ? __builtin_nontemporal_load(src + i + d * NT) : src[i + d * NT];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) acc ^= v[d];
    }
    for (; i < end; i += NT) acc ^= src[i];
    unsigned int v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v ^= __shfl_xor(v, off, 64);
    if ((threadIdx.x & 63) == 0) atomicXor(out + blockIdx.x, v);
}

// The same through buffer loads (the weight streams of the few-rows products are buffer loads) with the cache policy
// bits AUX of the instruction: 0 none, 1 sc0, 2 nt (non-temporal), 16 sc1, and their sums.
template <int AUX>
__global__ void __launch_bounds__(256)
probe_stream_buffer_kernel(const u32x4* __restrict__ src, int64_t pieces, unsigned int* __restrict__ out) {
    constexpr int NT = 256, DEPTH = 8;
    const int64_t per_block = (pieces + gridDim.x - 1) / gridDim.x;
    const int64_t begin = per_block * blockIdx.x, end = begin + per_block < pieces ? begin + per_block : pieces;
    // a workgroup's share is below 2 GiB: one buffer descriptor covers it
    const __amdgpu_buffer_rsrc_t res = __builtin_amdgcn_make_buffer_rsrc((void*)(src + begin), 0, (int)((end - begin) * 16), 0x00020000u);
    u32x4 acc = {0u, 0u, 0u, 0u};
    const int64_t count = end - begin;
    int64_t i = threadIdx.x;
    for (; i + (DEPTH - 1) * NT < count; i += DEPTH * NT) {
        u32x4 v[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) v[d] = __builtin_amdgcn_raw_buffer_load_b128(res, (unsigned)((i + d * NT) * 16), 0, AUX);
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) acc ^= v[d];
    }
    for (; i < count; i += NT) acc ^= __builtin_amdgcn_raw_buffer_load_b128(res, (unsigned)(i * 16), 0, AUX);
    unsigned int v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v ^= __shfl_xor(v, off, 64);
    if ((threadIdx.x & 63) == 0) atomicXor(out + blockIdx.x, v);
}

// The read pattern of a tiled matrix product's weight operand: the buffer is a matrix of rows of `row_bytes`; a
// workgroup owns 256 consecutive rows and walks them in steps of 128 bytes a row (2,048 loads of 16 bytes a step, two
// steps in flight).  SHARE workgroups own the same rows and take the steps in turns (SHARE = 1: each its own rows).
template <int SHARE>
__global__ void __launch_bounds__(256)
probe_tile_rows_kernel(const char* __restrict__ src, int row_groups, int row_bytes, unsigned int* __restrict__ out) {
    const int group = blockIdx.x / SHARE, turn = blockIdx.x % SHARE;
    if (group >= row_groups) return;
    const int steps = row_bytes / 128;
    const char* base = src + ((int64_t)group * 256 + (threadIdx.x >> 3)) * row_bytes + (threadIdx.x & 7) * 16;
    u32x4 acc = {0u, 0u, 0u, 0u};
    u32x4 a[8], b[8];
    auto fetch = [&](u32x4 (&to)[8], int step) {
#pragma unroll
        for (int pass = 0; pass < 8; ++pass)
            to[pass] = *(const u32x4*)(base + (int64_t)pass * 32 * row_bytes + (int64_t)step * 128);
    };
    int step = turn;
    if (step < steps) fetch(a, step);
    for (; step < steps; step += 2 * SHARE) {
        if (step + SHARE < steps) fetch(b, step + SHARE);
#pragma unroll
        for (int pass = 0; pass < 8; ++pass) acc ^= a[pass];
        if (step + 2 * SHARE < steps) fetch(a, step + 2 * SHARE);
        if (step + SHARE < steps) {
#pragma unroll
            for (int pass = 0; pass < 8; ++pass) acc ^= b[pass];
        }
    }
    unsigned int v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v ^= __shfl_xor(v, off, 64);
    if ((threadIdx.x & 63) == 0) atomicXor(out + (blockIdx.x & 1023), v);
}

// Every wavefront multiplies `iters` times four independent 32 x 32 x 16 bfloat16 products (32,768 flops each).
// dense: operands with every mantissa bit in use (hashed values in [-1, 1)), as a product of real activations and
// weights has them; otherwise small integers, most of whose bits are zero.  The part's clock under matrix
// instructions goes with what the operands toggle: the same loop runs a third slower on dense operands, and that is
// the rate a product can be held against.
__global__ void __launch_bounds__(512)
probe_mfma_kernel(int iters, int dense, float* __restrict__ out) {
    bf16x8 a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        if (dense) {
            unsigned ha = (threadIdx.x * 8u + e + blockIdx.x * 4099u) * 2654435761u, hb = (ha ^ 0x9e3779b9u) * 2246822519u;
            ha ^= ha >> 15; hb ^= hb >> 13;
            a[e] = (bf16)((float)(int)(ha & 0xffff) * (1.f / 32768.f) - 1.f);
            b[e] = (bf16)((float)(int)(hb & 0xffff) * (1.f / 32768.f) - 1.f);
        } else {
            a[e] = (bf16)(float)((threadIdx.x + e) & 3);
            b[e] = (bf16)(float)((threadIdx.x * 3 + e) & 1);
        }
    }
    f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int i = 0; i < iters; ++i) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
    }
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) sum += c0[r] + c1[r] + c2[r] + c3[r];
    if (sum == -1.f) out[0] = sum;          // never true: the products stay
}

// The launch shapes of the streaming read, so that the figure reported as the machine's own is the best of them and
// not what one arbitrary kernel happens to reach.
struct ProbeShape { const char* name; int threads, depth, nontemporal, blocks_per_unit; };
static const ProbeShape probe_shapes[] = {
    {"256 lanes x 4 loads, 8 workgroups a unit", 256, 4, 0, 8},
    {"256 lanes x 8 loads, 8 workgroups a unit", 256, 8, 0, 8},
    {"256 lanes x 16 loads, 4 workgroups a unit", 256, 16, 0, 4},
    {"512 lanes x 8 loads, 4 workgroups a unit", 512, 8, 0, 4},
    {"512 lanes x 8 loads, 2 workgroups a unit", 512, 8, 0, 2},
    {"256 lanes x 8 loads, non-temporal, 8 workgroups a unit", 256, 8, 1, 8},
    {"512 lanes x 16 loads, non-temporal, 4 workgroups a unit", 512, 16, 1, 4},
    // buffer loads of 256 lanes x 8, 8 workgroups a unit; `nontemporal` holds 100 + the cache policy bits
    {"buffer loads, no policy bits", 256, 8, 100, 8},
    {"buffer loads, sc0", 256, 8, 101, 8},
    {"buffer loads, nt", 256, 8, 102, 8},
    {"buffer loads, sc0 nt", 256, 8, 103, 8},
    {"buffer loads, sc1", 256, 8, 116, 8},
    {"buffer loads, sc1 nt", 256, 8, 118, 8},
    {"buffer loads, sc0 sc1 nt", 256, 8, 119, 8},
    // the weight operand of a tiled product: 256 rows of 7,168 bytes a workgroup, 128 bytes of each row a step
    // (`nontemporal` holds 200 + the workgroups that share a group of rows and take its steps in turns)
    {"tile rows: 256 rows x 128 bytes a step", 256, 2, 201, 0},
    {"tile rows, steps shared by 8 workgroups in turns", 256, 2, 208, 0},
};
#define PROBE_SHAPES ((int)(sizeof(probe_shapes) / sizeof(probe_shapes[0])))

extern "C" int somi_probe_stream_shapes() { return PROBE_SHAPES; }
extern "C" const char* somi_probe_stream_shape_name(int shape) {
    return shape >= 0 && shape < PROBE_SHAPES ? probe_shapes[shape].name : "";
}

// Workgroups of the streaming read in launch shape `shape`: what `out` must hold.
extern "C" int somi_probe_stream_blocks(int shape) {
    if (shape < 0 || shape >= PROBE_SHAPES) return 0;
    if (probe_shapes[shape].nontemporal >= 200) return 1024;
    return somi_units() * probe_shapes[shape].blocks_per_unit;
}

// Streams `bytes` (a multiple of 16, 16-byte aligned) from src once in launch shape `shape`.  out:
// [somi_probe_stream_blocks(shape)] words the caller zeroed.
extern "C" int somi_probe_stream_read(const void* src, int64_t bytes, int shape, unsigned int* out, hipStream_t stream) {
    SOMI_REQUIRE(src != nullptr && out != nullptr && bytes > 0 && bytes % 16 == 0 && (uintptr_t)src % 16 == 0,
                 "probe_stream_read: a 16-byte aligned buffer of a multiple of 16 bytes is needed");
    SOMI_REQUIRE(shape >= 0 && shape < PROBE_SHAPES, "probe_stream_read: launch shape %d (0 to %d)", shape, PROBE_SHAPES - 1);
    const ProbeShape& ps = probe_shapes[shape];
    const dim3 grid(somi_probe_stream_blocks(shape)), block(ps.threads);
    const u32x4* from = (const u32x4*)src;
    const int64_t pieces = bytes / 16;
#define SOMI_PROBE(NT, DEPTH, NTL)                                                                              \
    if (ps.threads == NT && ps.depth == DEPTH && ps.nontemporal == NTL) {                                        \
        hipLaunchKernelGGL((probe_stream_read_kernel<NT, DEPTH, NTL != 0>), grid, block, 0, stream, from, pieces, out); \
        SOMI_LAUNCH_CHECK("probe_stream_read");                                                                  \
        return 0;                                                                                                \
    }
    SOMI_PROBE(256, 4, 0) SOMI_PROBE(256, 8, 0) SOMI_PROBE(256, 16, 0) SOMI_PROBE(512, 8, 0)
    SOMI_PROBE(256, 8, 1) SOMI_PROBE(512, 16, 1)
#undef SOMI_PROBE
    if (ps.nontemporal >= 200) {
        // rows of 7,168 bytes (a K of 3,584 bfloat16): as many whole groups of 256 rows as the buffer holds
        const int row_bytes = 7168, share = ps.nontemporal - 200;
        const int groups = (int)(bytes / ((int64_t)row_bytes * 256));
        SOMI_REQUIRE(groups > 0, "probe_stream_read: the buffer holds no group of 256 rows");
        if (share == 1) hipLaunchKernelGGL((probe_tile_rows_kernel<1>), dim3(groups), block, 0, stream, (const char*)src, groups, row_bytes, out);
        else hipLaunchKernelGGL((probe_tile_rows_kernel<8>), dim3(groups * 8), block, 0, stream, (const char*)src, groups, row_bytes, out);
        SOMI_LAUNCH_CHECK("probe_stream_read");
        return 0;
    }
#define SOMI_PROBE_BUFFER(AUX)                                                                                   \
    if (ps.nontemporal == 100 + AUX) {                                                                           \
        SOMI_REQUIRE(bytes / grid.x < ((int64_t)1 << 31), "probe_stream_read: too many bytes a workgroup for a buffer descriptor"); \
        hipLaunchKernelGGL((probe_stream_buffer_kernel<AUX>), grid, block, 0, stream, from, pieces, out);        \
        SOMI_LAUNCH_CHECK("probe_stream_read");                                                                  \
        return 0;                                                                                                \
    }
    SOMI_PROBE_BUFFER(0) SOMI_PROBE_BUFFER(1) SOMI_PROBE_BUFFER(2) SOMI_PROBE_BUFFER(3) SOMI_PROBE_BUFFER(16)
    SOMI_PROBE_BUFFER(18) SOMI_PROBE_BUFFER(19)
#undef SOMI_PROBE_BUFFER
    return somi_fail("probe_stream_read: launch shape %d has no kernel", shape);
}

// Runs the products on every compute unit (two wavefronts per SIMD); returns the number of flops through *flops.
// dense: see probe_mfma_kernel.
extern "C" int somi_probe_mfma(int iters, int dense, float* out, double* flops, hipStream_t stream) {
    SOMI_REQUIRE(iters > 0 && out != nullptr, "probe_mfma: bad arguments");
    int device = 0;
    hipDeviceProp_t prop;
    SOMI_REQUIRE(hipGetDevice(&device) == hipSuccess && hipGetDeviceProperties(&prop, device) == hipSuccess,
                 "probe_mfma: no device properties");
    const int blocks = prop.multiProcessorCount;
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(512), 0, stream, iters, dense, out);
    SOMI_LAUNCH_CHECK("probe_mfma");
    if (flops != nullptr) *flops = (double)blocks * 8.0 * (double)iters * 4.0 * 32768.0;
    return 0;
}
