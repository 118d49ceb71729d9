// Plain causal attention over cache pages for any mix of prompt portions and decoded tokens.
//
// Reference formulas: somi_inference/models/qwen2.py:158-186 (scores = q.k * D^-0.5, causal mask,
// float32 softmax, weights . v; query head h uses key/value head h // (nq / nkv)) and
// somi_inference/core/paged_attention.py:352-413 (walk the block table page by page with a running
// max, running sum and rescaled output; positions >= seq_len are masked).
//
// One workgroup per (token, query head).  A token at position p of its request attends to the
// cached keys at positions max(0, p - window + 1) .. p of the same request (window == 0: all),
// which include the keys this step wrote before the launch.  Keys are walked in tiles of NT
// aligned to absolute positions, so the arithmetic for a (request, position) is the same
// whatever portion or batch the token arrives in.  Everything is float32.
#include "common.h"

template <typename T, int NT>
__global__ void __launch_bounds__(NT)
paged_attention_plain_kernel(const T* __restrict__ q, int64_t q_stride, const T* __restrict__ kc,
                             const T* __restrict__ vc, const int* __restrict__ block_table, int max_blocks,
                             const int* __restrict__ token_entry, const int* __restrict__ positions, int nq,
                             int nkv, int D, int page_size, int window, float scale, T* __restrict__ out) {
    extern __shared__ float smem[];
    float* qs = smem;                          // [D]
    float* ps = qs + ((D + 1) & ~1);           // [NT] softmax weights of the tile
    float* red = ps + NT;                      // [16]
    int64_t* rowoff = (int64_t*)(red + 16);    // [NT] element offset of each key row of the tile
    int64_t* coloff = rowoff + NT;             // [NT] element offset of each value column (V is [.., D, page_size])

    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int e = token_entry[t];
    const int p = positions[t];
    const int kvh = h / (nq / nkv);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* table = block_table + (int64_t)e * max_blocks;

    for (int d = tid; d < D; d += NT) qs[d] = to_float(q[(int64_t)t * q_stride + (int64_t)h * D + d]);

    float m = -INFINITY, l = 0.f;
    float acc[2] = {0.f, 0.f};                 // output dims tid and tid + NT (D <= 2 * NT)

    for (int tile = lo / NT; tile <= p / NT; ++tile) {
        const int pos = tile * NT + tid;
        const bool valid = pos >= lo && pos <= p;
        __syncthreads();                        // qs ready; previous tile's ps/rowoff no longer read
        float s = -INFINITY;
        if (valid) {
            const int64_t page = table[pos / page_size];
            const int64_t off = ((page * nkv + kvh) * page_size + pos % page_size) * (int64_t)D;
            rowoff[tid] = off;
            coloff[tid] = (page * nkv + kvh) * (int64_t)D * page_size + pos % page_size;
            const T* kr = kc + off;
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_float(kr[d]), dot);
            s = dot * scale;
        }
        const float tile_max = block_max<NT>(s, red);
        const float m_new = fmaxf(m, tile_max);
        const float corr = expf(m - m_new);     // exp(-inf) = 0 on the first tile
        const float w = valid ? expf(s - m_new) : 0.f;
        ps[tid] = w;
        const float tile_sum = block_sum<NT>(w, red);
        l = l * corr + tile_sum;
        m = m_new;
        __syncthreads();                        // ps and rowoff visible
        const int j0 = (lo > tile * NT ? lo : tile * NT) - tile * NT;
        const int j1 = (p < tile * NT + NT - 1 ? p : tile * NT + NT - 1) - tile * NT;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int d = tid + r * NT;
            if (d < D) {
                float a = acc[r] * corr;
                for (int j = j0; j <= j1; ++j) a = fmaf(ps[j], to_float(vc[coloff[j] + (int64_t)d * page_size]), a);
                acc[r] = a;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int d = tid + r * NT;
        if (d < D) out[((int64_t)t * nq + h) * D + d] = from_float<T>(acc[r] / l);
    }
}

// q: token t's head h starts at q + t * q_stride + h * D.  k_cache: [num_pages, nkv, page_size, D];
// v_cache: [num_pages, nkv, D, page_size].
// block_table: [n_entries, max_blocks] int32 page ids of each entry's request (pages a window has passed
// may hold -1; they are never read).  token_entry, positions: [n_tokens] int32.  out: [n_tokens, nq * D].
extern "C" int somi_paged_attention_plain(const void* q, int dtype, int64_t q_stride, const void* k_cache,
                                          const void* v_cache, const int* block_table, int max_blocks,
                                          const int* token_entry, const int* positions, int n_tokens, int nq,
                                          int nkv, int D, int page_size, int window, float scale, void* out,
                                          hipStream_t stream) {
    constexpr int NT = 128;
    SOMI_REQUIRE(n_tokens >= 0 && nq > 0 && nkv > 0 && D > 0 && page_size > 0 && max_blocks > 0,
                 "paged_attention: bad sizes");
    SOMI_REQUIRE(nq % nkv == 0, "paged_attention: num_q_heads (%d) must be divisible by num_kv_heads (%d)", nq, nkv);
    SOMI_REQUIRE(D <= 2 * NT, "paged_attention: head_dim %d is larger than the supported %d", D, 2 * NT);
    SOMI_REQUIRE(window >= 0, "paged_attention: window must be >= 0");
    SOMI_REQUIRE(nq <= 65535, "paged_attention: too many heads");
    if (n_tokens == 0) return 0;
    const dim3 grid(n_tokens, nq);
    const size_t smem = (size_t)(((D + 1) & ~1) + NT + 16) * sizeof(float) + 2 * NT * sizeof(int64_t);
    if (dtype == SOMI_F32)
        hipLaunchKernelGGL((paged_attention_plain_kernel<float, NT>), grid, dim3(NT), smem, stream, (const float*)q,
                           q_stride, (const float*)k_cache, (const float*)v_cache, block_table, max_blocks,
                           token_entry, positions, nq, nkv, D, page_size, window, scale, (float*)out);
    else if (dtype == SOMI_BF16)
        hipLaunchKernelGGL((paged_attention_plain_kernel<bf16, NT>), grid, dim3(NT), smem, stream, (const bf16*)q,
                           q_stride, (const bf16*)k_cache, (const bf16*)v_cache, block_table, max_blocks,
                           token_entry, positions, nq, nkv, D, page_size, window, scale, (bf16*)out);
    else
        return somi_fail("paged_attention: unknown dtype %d", dtype);
    SOMI_LAUNCH_CHECK("paged_attention_plain");
    return 0;
}
