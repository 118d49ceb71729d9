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

// Reads `pieces` 16-byte pieces once, every workgroup a contiguous share in steps of its 256 lanes, four loads in
// flight a lane; the exclusive-or of everything read goes to out[blockIdx.x] so that no load can be dropped.
__global__ void __launch_bounds__(256)
probe_stream_read_kernel(const u32x4* __restrict__ src, int64_t pieces, unsigned int* __restrict__ out) {
    const int64_t per_block = (pieces + gridDim.x - 1) / gridDim.x;
    const int64_t begin = per_block * blockIdx.x, end = begin + per_block < pieces ? begin + per_block : pieces;
    u32x4 acc = {0u, 0u, 0u, 0u};
    int64_t i = begin + threadIdx.x;
    for (; i + 3 * 256 < end; i += 4 * 256) {
        const u32x4 a = src[i], b = src[i + 256], c = src[i + 512], d = src[i + 768];
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < end; i += 256) acc ^= src[i];
    unsigned int v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v ^= __shfl_xor(v, off, 64);
    if ((threadIdx.x & 63) == 0) atomicXor(out + blockIdx.x, v);
}

// Every wavefront multiplies `iters` times four independent 32 x 32 x 16 bfloat16 products (32,768 flops each).
__global__ void __launch_bounds__(512)
probe_mfma_kernel(int iters, float* __restrict__ out) {
    bf16x8 a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = (bf16)(float)((threadIdx.x + e) & 3);
        b[e] = (bf16)(float)((threadIdx.x * 3 + e) & 1);
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

// Streams `bytes` (a multiple of 16, 16-byte aligned) from src once.  out: [blocks] words the caller zeroed,
// blocks = somi_probe_stream_blocks().
extern "C" int somi_probe_stream_blocks() {
    int device = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess) return 2048;
    return prop.multiProcessorCount * 8;
}

extern "C" int somi_probe_stream_read(const void* src, int64_t bytes, unsigned int* out, hipStream_t stream) {
    SOMI_REQUIRE(src != nullptr && out != nullptr && bytes > 0 && bytes % 16 == 0 && (uintptr_t)src % 16 == 0,
                 "probe_stream_read: a 16-byte aligned buffer of a multiple of 16 bytes is needed");
    hipLaunchKernelGGL(probe_stream_read_kernel, dim3(somi_probe_stream_blocks()), dim3(256), 0, stream,
                       (const u32x4*)src, bytes / 16, out);
    SOMI_LAUNCH_CHECK("probe_stream_read");
    return 0;
}

// Runs the products on every compute unit (two wavefronts per SIMD); returns the number of flops through *flops.
extern "C" int somi_probe_mfma(int iters, float* out, double* flops, hipStream_t stream) {
    SOMI_REQUIRE(iters > 0 && out != nullptr, "probe_mfma: bad arguments");
    int device = 0;
    hipDeviceProp_t prop;
    SOMI_REQUIRE(hipGetDevice(&device) == hipSuccess && hipGetDeviceProperties(&prop, device) == hipSuccess,
                 "probe_mfma: no device properties");
    const int blocks = prop.multiProcessorCount;
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(512), 0, stream, iters, out);
    SOMI_LAUNCH_CHECK("probe_mfma");
    if (flops != nullptr) *flops = (double)blocks * 8.0 * (double)iters * 4.0 * 32768.0;
    return 0;
}
