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

#define ROPE_THREADS 256
#define ROPE_MAX_HALF 256                      // rotary_dim / 2 at most

// One workgroup per (token, group of heads): cos and sin of the token's angles are computed once into LDS
// and serve every head of the group; the group's (head, channel pair) items are dealt to the threads.
template <typename T>
struct __attribute__((aligned(16))) Pack8 { T v[8]; };      // eight bfloat16: one 16-byte access

template <typename T, bool VEC8>
__global__ void __launch_bounds__(ROPE_THREADS)
rope_kv_store_kernel(T* __restrict__ qkv, int64_t row_stride, const int* __restrict__ positions,
                     const int* __restrict__ slots, const float* __restrict__ inv_freq, int rot_half,
                     int nq, int nkv, int D, T* __restrict__ kc, T* __restrict__ vc, int page_size,
                     int heads_per_block) {
    __shared__ float cs[2][ROPE_MAX_HALF];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int h0 = blockIdx.y * heads_per_block;               // heads 0..nq-1: q, then nkv k heads, then nkv v heads
    const int h1 = min(h0 + heads_per_block, nq + 2 * nkv);
    T* row = qkv + (int64_t)t * row_stride;
    if (inv_freq) {
        const float pos = (float)positions[t];
        for (int j = tid; j < rot_half; j += ROPE_THREADS) {
            const float angle = pos * inv_freq[j];
            cs[0][j] = cosf(angle);
            cs[1][j] = sinf(angle);
        }
    }
    __syncthreads();
    const int slot = nkv > 0 ? slots[t] : -1;                  // -1: a token without a cache slot (padding)
    const int64_t page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;

    // q (in place) and k (into its page): rotate the pairs (j, j + rot_half)
    const int rot0 = h0, rot1 = min(h1, nq + nkv);
    if (VEC8 && rot_half > 0) {
        // eight neighbouring pairs per thread: 16-byte loads and stores (the launcher checked the alignment)
        const int groups = rot_half / 8;
        for (int item = tid; item < (rot1 - rot0) * groups; item += ROPE_THREADS) {
            const int hh = rot0 + item / groups, j = (item % groups) * 8;
            const T* src = row + (int64_t)hh * D + j;
            T* dst = row + (int64_t)hh * D + j;
            if (hh >= nq) {
                if (slot < 0) continue;
                dst = kc + ((page * nkv + (hh - nq)) * page_size + off) * D + j;
            }
            Pack8<T> lo = *reinterpret_cast<const Pack8<T>*>(src), hi = *reinterpret_cast<const Pack8<T>*>(src + rot_half);
            Pack8<T> first, second;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x1 = to_float(lo.v[i]), x2 = to_float(hi.v[i]);
                const float c = cs[0][j + i], sn = cs[1][j + i];
                first.v[i] = from_float<T>(x1 * c - x2 * sn);
                second.v[i] = from_float<T>(x2 * c + x1 * sn);
            }
            *reinterpret_cast<Pack8<T>*>(dst) = first;
            *reinterpret_cast<Pack8<T>*>(dst + rot_half) = second;
        }
    } else if (rot_half > 0)
        for (int item = tid; item < (rot1 - rot0) * rot_half; item += ROPE_THREADS) {
            const int hh = rot0 + item / rot_half, j = item % rot_half;
            const T* src = row + (int64_t)hh * D;
            T* dst = row + (int64_t)hh * D;
            if (hh >= nq) {
                if (slot < 0) continue;
                dst = kc + ((page * nkv + (hh - nq)) * page_size + off) * D;
            }
            const float x1 = to_float(src[j]), x2 = to_float(src[j + rot_half]);
            const float c = cs[0][j], sn = cs[1][j];
            dst[j] = from_float<T>(x1 * c - x2 * sn);
            dst[j + rot_half] = from_float<T>(x2 * c + x1 * sn);
        }
    // k: the channels past the rotated ones go to the page as they are
    const int k0 = max(h0, nq), k1 = min(h1, nq + nkv), rest = D - 2 * rot_half;
    if (slot >= 0 && rest > 0)
        for (int item = tid; item < (k1 - k0) * rest; item += ROPE_THREADS) {
            const int hh = k0 + item / rest, d = 2 * rot_half + item % rest;
            kc[((page * nkv + (hh - nq)) * page_size + off) * D + d] = row[(int64_t)hh * D + d];
        }
    // v: into its page, transposed
    const int v0 = max(h0, nq + nkv), v1 = h1;
    if (slot >= 0)
        for (int item = tid; item < (v1 - v0) * D; item += ROPE_THREADS) {
            const int hh = v0 + item / D, d = item % D;
            vc[((page * nkv + (hh - nq - nkv)) * (int64_t)D + d) * page_size + off] = row[(int64_t)hh * D + d];
        }
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
    SOMI_REQUIRE(rotary_dim / 2 <= ROPE_MAX_HALF, "rope_kv_store: rotary_dim %d is more than %d", rotary_dim,
                 2 * ROPE_MAX_HALF);
    if (n_tokens == 0 || nq + 2 * nkv == 0) return 0;
    // about two thousand workgroups: one head each for a few tokens, all heads of a token for long portions
    const int heads = nq + 2 * nkv;
    const int heads_per_block = max(1, min(heads, (int)(((int64_t)n_tokens * heads + 2047) / 2048)));
    const dim3 grid(n_tokens, ceil_div(heads, heads_per_block));
    const int rot_half = inv_freq ? rotary_dim / 2 : 0;
    // the 16-byte path of bfloat16: every head, half and row starts at a multiple of eight elements
    const bool vec8 = dtype == SOMI_BF16 && rot_half % 8 == 0 && D % 8 == 0 && row_stride % 8 == 0 &&
                      (uintptr_t)qkv % 16 == 0 && (nkv == 0 || (uintptr_t)k_cache % 16 == 0);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL((rope_kv_store_kernel<float, false>), grid, dim3(ROPE_THREADS), 0, stream, (float*)qkv,
                           row_stride, positions, slots, inv_freq, rot_half, nq, nkv, D, (float*)k_cache,
                           (float*)v_cache, page_size, heads_per_block);
    else if (dtype == SOMI_BF16 && vec8)
        hipLaunchKernelGGL((rope_kv_store_kernel<bf16, true>), grid, dim3(ROPE_THREADS), 0, stream, (bf16*)qkv, row_stride,
                           positions, slots, inv_freq, rot_half, nq, nkv, D, (bf16*)k_cache, (bf16*)v_cache,
                           page_size, heads_per_block);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL((rope_kv_store_kernel<bf16, false>), grid, dim3(ROPE_THREADS), 0, stream, (bf16*)qkv, row_stride,
                           positions, slots, inv_freq, rot_half, nq, nkv, D, (bf16*)k_cache, (bf16*)v_cache,
                           page_size, heads_per_block);
    else
        return somi_fail("rope_kv_store: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("rope_kv_store");
    return 0;
}
