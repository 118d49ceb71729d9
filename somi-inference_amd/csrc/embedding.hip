// Embedding gather: h[t, :] = E[id[t], :], written as float32 into the residual stream.
// Reference: somi_inference/models/qwen2.py:360,382 (nn.Embedding lookup).
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
embedding_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out,
                 int hidden, int vocab) {
    const int t = blockIdx.x;
    int id = ids[t];
    // Ids are range-checked on the host before the launch; the clamp only
    // keeps a stray value from reading outside the table.
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const T* row = table + (int64_t)id * hidden;
    float* dst = out + (int64_t)t * hidden;
    for (int i = threadIdx.x; i < hidden; i += 256) dst[i] = to_float(row[i]);
}

extern "C" int somi_embedding(const void* table, int dtype, const int* ids, float* out, int n_tokens,
                              int hidden, int vocab, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0, "embedding: bad sizes n=%d hidden=%d vocab=%d",
                 n_tokens, hidden, vocab);
    if (n_tokens == 0) return 0;
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(embedding_kernel<float>, dim3(n_tokens), dim3(256), 0, stream,
                           (const float*)table, ids, out, hidden, vocab);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(embedding_kernel<bf16>, dim3(n_tokens), dim3(256), 0, stream,
                           (const bf16*)table, ids, out, hidden, vocab);
    else
        return somi_fail("embedding: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("embedding");
    return 0;
}

// out[r, :] = src[rows[r], :] for float32 rows (selects the positions whose logits are wanted).
__global__ void __launch_bounds__(256)
gather_rows_kernel(const float* __restrict__ src, const int* __restrict__ rows, float* __restrict__ out,
                   int width) {
    const float* s = src + (int64_t)rows[blockIdx.x] * width;
    float* d = out + (int64_t)blockIdx.x * width;
    for (int i = threadIdx.x; i < width; i += 256) d[i] = s[i];
}

extern "C" int somi_gather_rows_f32(const float* src, const int* rows, float* out, int n_rows, int width,
                                    hipStream_t stream) {
    SOMI_REQUIRE(n_rows >= 0 && width > 0, "gather_rows: bad sizes rows=%d width=%d", n_rows, width);
    if (n_rows == 0) return 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(n_rows), dim3(256), 0, stream, src, rows, out, width);
    SOMI_LAUNCH_CHECK("gather_rows");
    return 0;
}
