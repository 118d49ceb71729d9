// Rotary position encoding of q and k, fused with the write of k and v into cache pages.
//
// Reference: somi_inference/models/qwen2.py:72-81 (inv_freq[j] = 1 / theta^(2j/D), freq = p * inv_freq,
// cos/sin of cat(freq, freq)), :95-113 (rotate_half([x1, x2]) = [-x2, x1]; x' = x*cos + rotate_half(x)*sin,
// on q and k only) and somi_inference/core/paged_attention.py:246-292 (k is cached after rotation; a token
// lands in page[pos // block_size] at slot pos % block_size).
//
// The angle p * inv_freq[j] and its cos/sin are float32 whatever the storage type; inv_freq comes
// from the host as a float32 table so both engines and the plain implementation share it.
// Cache layout per layer: K [num_pages, n_kv_heads, page_size, head_dim]; V is kept transposed inside
// a page, [num_pages, n_kv_heads, head_dim, page_size], so that the attention kernels read consecutive
// positions of one channel with one load (the operand layout of the matrix cores for P.V).
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(64)
rope_kv_store_kernel(T* __restrict__ qkv, int64_t row_stride, const int* __restrict__ positions,
                     const int* __restrict__ slots, const float* __restrict__ inv_freq, int rot_half,
                     int nq, int nkv, int D, T* __restrict__ kc, T* __restrict__ vc, int page_size) {
    const int t = blockIdx.x;
    const int hh = blockIdx.y;                 // 0..nq-1: q heads, then nkv k heads, then nkv v heads
    T* src = qkv + (int64_t)t * row_stride + (int64_t)hh * D;
    const float pos = (float)positions[t];

    T* dst = nullptr;                          // cache row, when this head is a k or v head
    if (hh >= nq) {
        const int slot = slots[t];
        if (slot < 0) return;                  // a token without a cache slot (padding)
        const bool is_v = hh >= nq + nkv;
        const int kvh = hh - nq - (is_v ? nkv : 0);
        const int64_t page = slot / page_size, off = slot % page_size;
        if (is_v) {
            T* col = vc + (page * nkv + kvh) * (int64_t)D * page_size + off;
            for (int d = threadIdx.x; d < D; d += 64) col[(int64_t)d * page_size] = src[d];
            return;
        }
        dst = kc + ((page * nkv + kvh) * page_size + off) * D;
    }
    T* q_or_k = dst ? dst : src;               // q is rotated in place, k goes to its page
    for (int j = threadIdx.x; j < rot_half; j += 64) {
        const float x1 = to_float(src[j]), x2 = to_float(src[j + rot_half]);
        float c = 1.f, s = 0.f;
        if (inv_freq) {
            const float angle = pos * inv_freq[j];
            c = cosf(angle);
            s = sinf(angle);
        }
        q_or_k[j] = from_float<T>(x1 * c - x2 * s);
        q_or_k[j + rot_half] = from_float<T>(x2 * c + x1 * s);
    }
    if (dst)                                   // pass-through tail of a partly rotated head
        for (int d = 2 * rot_half + threadIdx.x; d < D; d += 64) dst[d] = src[d];
}

// qkv: [n_tokens, row_stride] with q heads, k heads, v heads side by side (row_stride >= (nq+2nkv)*D).
// positions, slots: [n_tokens] int32; slot = page * page_size + offset, or -1 for "do not store".
// inv_freq: [rotary_dim/2] float32, or null for no rotation.  With nkv == 0 only q is rotated.
extern "C" int somi_rope_kv_store(void* qkv, int dtype, int64_t row_stride, const int* positions, const int* slots,
                                  const float* inv_freq, int rotary_dim, int n_tokens, int nq, int nkv, int D,
                                  void* k_cache, void* v_cache, int page_size, hipStream_t stream) {
    SOMI_REQUIRE(n_tokens >= 0 && nq >= 0 && nkv >= 0 && D > 0, "rope_kv_store: bad sizes");
    SOMI_REQUIRE(rotary_dim >= 0 && rotary_dim <= D && rotary_dim % 2 == 0,
                 "rope_kv_store: rotary_dim %d must be even and <= head_dim %d", rotary_dim, D);
    SOMI_REQUIRE(row_stride >= (int64_t)(nq + 2 * nkv) * D, "rope_kv_store: row stride %lld too small",
                 (long long)row_stride);
    SOMI_REQUIRE(nkv == 0 || (k_cache && v_cache && slots && page_size > 0),
                 "rope_kv_store: cache pointers, slots and page size are needed when k/v heads are given");
    SOMI_REQUIRE(nq + 2 * nkv <= 65535, "rope_kv_store: too many heads");
    if (n_tokens == 0 || nq + 2 * nkv == 0) return 0;
    const dim3 grid(n_tokens, nq + 2 * nkv);
    const int rot_half = inv_freq ? rotary_dim / 2 : 0;
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL(rope_kv_store_kernel<float>, grid, dim3(64), 0, stream, (float*)qkv, row_stride,
                           positions, slots, inv_freq, rot_half, nq, nkv, D, (float*)k_cache, (float*)v_cache,
                           page_size);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL(rope_kv_store_kernel<bf16>, grid, dim3(64), 0, stream, (bf16*)qkv, row_stride,
                           positions, slots, inv_freq, rot_half, nq, nkv, D, (bf16*)k_cache, (bf16*)v_cache,
                           page_size);
    else
        return somi_fail("rope_kv_store: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("rope_kv_store");
    return 0;
}
