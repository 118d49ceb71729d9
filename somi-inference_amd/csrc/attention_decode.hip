// Paged grouped-query attention for decoded tokens and short portions, bfloat16, on the matrix cores.
//
// Reference: somi_inference/core/paged_attention.py:352-413 (walk the block table with a running max,
// running sum and rescaled output; float32 softmax state; weights cast to the value dtype before P.V) and
// its Triton twin core/paged_attention_triton.py:29-150, which launches one program per (sequence, query
// head) and so reads every key and value nq/nkv times.  Here one workgroup serves all query heads that
// share a key/value head, and the keys of a long context are split over workgroups so that a few
// requests still fill 256 compute units:
//   grid = (token, kv head x blocks of 16 query heads, split of the context)
//   a wavefront takes 16-key tiles (aligned to absolute positions) of its split in turn;
//   S^T[key, head] = K[key, :] . Q^T   (v_mfma_f32_16x16x32_bf16; K rows are the A operand, read 16 B per lane)
//   online softmax per head over the tile in float32 (the four keys a lane holds, then across lane groups)
//   O^T[d, head] += V^T[d, key] . P^T (v_mfma_f32_16x16x16_bf16; S^T comes out of the first product in
//                   exactly the B-operand layout, and V is stored transposed inside a page so a lane reads
//                   four consecutive keys of one channel with one 8-byte load)
// The wavefronts of a workgroup are merged through LDS; with several splits the workgroup writes
// (max, sum, unnormalised output) to a workspace and a second kernel merges the splits in split order.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short short4_t;

// Four values (keys vpos .. vpos + 3 of one channel) with those outside [lo, hi] set to zero.  A masked key has the
// weight 0, but 0 x NaN is NaN: what lies beyond a request's tokens in a page that is used again, or before its
// window, must not reach the products, whatever it holds.
__device__ __forceinline__ short4_t keep_visible(short4_t v, int vpos, int lo, int hi) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
        if (vpos + e < lo || vpos + e > hi) v[e] = 0;
    return v;
}
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 ld8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ short4_t ld4(const bf16* p) { return *reinterpret_cast<const short4_t*>(p); }
// The same for keys and values: a decode step reads each of them once, so the loads tell the caches not to keep the
// lines (a streaming read measures 6.6 TB/s that way against 5.9 on an MI355X).
typedef __attribute__((ext_vector_type(4))) unsigned int decode_u32x4;
__device__ __forceinline__ bf16x8 ld8_once(const bf16* p) {
    union { decode_u32x4 raw; bf16x8 values; } u;
    u.raw = __builtin_nontemporal_load(reinterpret_cast<const decode_u32x4*>(p));
    return u.values;
}
__device__ __forceinline__ short4_t ld4_once(const bf16* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const short4_t*>(p));
}
// Four elements in the lower half of an eight-wide operand, zeros above.
__device__ __forceinline__ bf16x8 half_step(const bf16* p) {
    union { bf16x8 wide; short4_t half[2]; } u;
    u.half[0] = ld4(p);
    u.half[1] = short4_t{0, 0, 0, 0};
    return u.wide;
}

// The keys of split `split` of a token at position p that sees keys from lo on: the visible range (from the
// 32-key tile that holds lo) cut into num_splits equal parts of a multiple of 16 keys, at most split_len each.
// The parts follow the token's own range, not the longest context the launch was sized for, so a launch with
// more splits than a short context needs (a captured step serves contexts up to its block tables' width) still
// gives every workgroup a share of the keys.
__device__ __forceinline__ void decode_split_range(int p, int lo, int split, int split_len, int num_splits, int& begin,
                                                   int& end) {
    const int base = lo & ~31;
    const int span = p - base + 1;
    int len = ((span + num_splits - 1) / num_splits + 15) & ~15;
    len = len < split_len ? len : split_len;
    const int first = base + split * len;
    begin = lo > first ? lo : first;
    end = p < first + len - 1 ? p : first + len - 1;
}

template <int DT>
__global__ void __launch_bounds__(256)
attention_decode_kernel(const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ kc,
                        const bf16* __restrict__ vc, const int* __restrict__ block_table, int max_blocks,
                        const int* __restrict__ token_list, const int* __restrict__ token_entry,
                        const int* __restrict__ positions, int nq, int nkv, int page_size, int window, float scale,
                        int split_len, int num_splits, bf16* __restrict__ out, float* __restrict__ part_acc,
                        float* __restrict__ part_ml) {
    constexpr int D = DT * 16;
    extern __shared__ float lds[];
    const int waves = blockDim.x >> 6;
    float* lds_acc = lds;                                  // [waves][DT][64][4]
    float* lds_m = lds + waves * DT * 256;                 // [waves][16]
    float* lds_l = lds_m + waves * 16;                     // [waves][16]

    const int ti = blockIdx.x;
    const int t = token_list ? token_list[ti] : ti;
    const int G = nq / nkv, HB = (G + 15) / 16;
    const int kvh = blockIdx.y / HB, hb = blockIdx.y % HB;
    const int split = blockIdx.z;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;

    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* table = block_table + (int64_t)token_entry[t] * max_blocks;
    int begin, end;                                  // this split's keys, inclusive
    decode_split_range(p, lo, split, split_len, num_splits, begin, end);

    const int hloc = hb * 16 + r;
    const int head = kvh * G + (hloc < G ? hloc : G - 1);
    const bf16* qrow = q + (int64_t)t * q_stride + (int64_t)head * D;
    // The head size is walked in 32-wide steps; an odd number of 16-wide tiles leaves a last step whose
    // upper half is zero in both operands.  (All products of the chain are the same instruction: a
    // 16x16x16 product that takes the result of a 16x16x32 one as its addend straight away, without an
    // instruction in between, has been seen to read it too early.)
    constexpr int QK_STEPS = (DT + 1) / 2;
    bf16x8 qf[QK_STEPS];
#pragma unroll
    for (int c = 0; c < DT / 2; ++c) qf[c] = ld8(qrow + c * 32 + g * 8);
    if (DT & 1) qf[QK_STEPS - 1] = half_step(qrow + (DT - 1) * 16 + g * 4);

    float m_run = -INFINITY, l_run = 0.f;
    f32x4 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (begin <= end) {
        for (int tile = begin / 16 + wave; tile <= end / 16; tile += waves) {
            const int j0 = tile * 16;
            // keys: lane reads row j0 + r (an address inside the split even where the key is masked)
            int pos = j0 + r;
            pos = pos < begin ? begin : (pos > end ? end : pos);
            const int64_t kpage = table[pos / page_size];
            const bf16* krow = kc + ((kpage * nkv + kvh) * page_size + pos % page_size) * (int64_t)D;
            // values: lane reads channel dt * 16 + r at keys j0 + 4 g .. + 3 (one page: page_size % 4 == 0)
            int vpos = j0 + g * 4;
            const int vlo = begin & ~3, vhi = end & ~3;
            vpos = vpos < vlo ? vlo : (vpos > vhi ? vhi : vpos);
            const int64_t vpage = table[vpos / page_size];
            const bf16* vbase = vc + (vpage * nkv + kvh) * (int64_t)D * page_size + vpos % page_size;
            // all loads of the tile are issued before the first product
            bf16x8 kf[QK_STEPS];
            short4_t vf[DT];
#pragma unroll
            for (int c = 0; c < DT / 2; ++c) kf[c] = ld8(krow + c * 32 + g * 8);
            if (DT & 1) kf[QK_STEPS - 1] = half_step(krow + (DT - 1) * 16 + g * 4);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) vf[dt] = ld4(vbase + (int64_t)(dt * 16 + r) * page_size);
            if (vpos == vlo || vpos == vhi) {          // the groups that hold the first and the last visible key
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) vf[dt] = keep_visible(vf[dt], vpos, begin, end);
            }
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < QK_STEPS; ++c) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[c], qf[c], s, 0, 0, 0);
            // s[i] = S[key j0 + 4 g + i][head r]
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int pj = j0 + g * 4 + i;
                s[i] = (pj >= begin && pj <= end) ? s[i] * scale : -INFINITY;
                mx = fmaxf(mx, s[i]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run, mx);           // finite: every tile holds a visible key
            const float corr = expf(m_run - m_new);
            float pr[4], sum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pr[i] = expf(s[i] - m_new);
                sum += pr[i];
            }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            l_run = l_run * corr + sum;
            m_run = m_new;
            bf16x4 pb = {(bf16)pr[0], (bf16)pr[1], (bf16)pr[2], (bf16)pr[3]};
            const short4_t pf = *reinterpret_cast<short4_t*>(&pb);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                acc[dt] *= corr;
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[dt], pf, acc[dt], 0, 0, 0);
            }
        }
    }

    // merge the wavefronts: acc[dt][i] = O^T[d = dt * 16 + 4 g + i][head r]
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        *reinterpret_cast<f32x4*>(lds_acc + ((wave * DT + dt) * 64 + lane) * 4) = acc[dt];
    if (g == 0) {
        lds_m[wave * 16 + r] = m_run;
        lds_l[wave * 16 + r] = l_run;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < DT * 256; idx += blockDim.x) {
        const int dt = idx >> 8, l = (idx >> 2) & 63, i = idx & 3;
        const int hr = l & 15;
        const int hl = hb * 16 + hr;
        if (hl >= G) continue;
        float m_all = -INFINITY;
        for (int w = 0; w < waves; ++w) m_all = fmaxf(m_all, lds_m[w * 16 + hr]);
        float total = 0.f, l_all = 0.f;
        if (m_all > -INFINITY) {
            for (int w = 0; w < waves; ++w) {
                const float f = expf(lds_m[w * 16 + hr] - m_all);
                total += lds_acc[w * DT * 256 + idx] * f;
                l_all += lds_l[w * 16 + hr] * f;
            }
        }
        const int d = dt * 16 + (l >> 4) * 4 + i;
        const int hq = kvh * G + hl;
        if (num_splits == 1) {
            out[((int64_t)t * nq + hq) * D + d] = (bf16)(total / l_all);
        } else {
            const int64_t slot = ((int64_t)ti * nq + hq) * num_splits + split;
            part_acc[slot * D + d] = total;
            if (dt == 0 && (l >> 4) == 0 && i == 0) {
                part_ml[slot * 2] = m_all;
                part_ml[slot * 2 + 1] = l_all;
            }
        }
    }
}

// The same with the keys and values of a split staged through LDS, 32 keys at a time: all 256 threads
// fetch the next 32 keys and values into registers while the current ones are used from LDS (many bytes
// in flight per workgroup, which is what a bandwidth-bound kernel needs).  Every wavefront computes the
// scores and the softmax of the 32 keys (a few products), then applies the weights to its own quarter of
// the head's channels, so the output needs no merge across wavefronts.
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
// Maxima of scores, which are never NaN (keys that must not be seen are -inf): the bare instructions, without
// the quieting of signalling NaNs that fmaxf adds to each operand.
__device__ __forceinline__ float max2(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float lanes4_max(float v) {       // over lanes l, l ^ 16, l ^ 32, l ^ 48
    u32x2 a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = max2(__uint_as_float(a[0]), __uint_as_float(a[1]));
    u32x2 b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return max2(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float lanes4_sum(float v) {
    u32x2 a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    u32x2 b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Pages of a split that the LDS copy of the block table holds: a table of 512 pages (8,192 keys in pages of 16, what a
// captured step of requests at 4,096 to 8,192 tokens allows) is one split, with four workgroups of head size 128 still
// fitting a compute unit's LDS (38 KB each).
#define DECODE_LDS_PAGES 768
template <int DT>
__global__ void __launch_bounds__(256)
attention_decode_lds_kernel(const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ kc,
                            const bf16* __restrict__ vc, const int* __restrict__ block_table, int max_blocks,
                            const int* __restrict__ token_list, const int* __restrict__ token_entry,
                            const int* __restrict__ positions, int nq, int nkv, int page_size, int window,
                            float scale, int split_len, int num_splits, bf16* __restrict__ out,
                            float* __restrict__ part_acc, float* __restrict__ part_ml) {
    constexpr int D = DT * 16;
    constexpr int QK_STEPS = (DT + 1) / 2;
    constexpr int KROW = D + 8, VROW = 32 + 4;               // padded LDS rows, in elements
    constexpr int K_CHUNKS = 32 * D / 8;                     // 16-byte pieces of a 32-key tile
    constexpr int K_PER_THREAD = (K_CHUNKS + 255) / 256;
    constexpr int V_PER_THREAD = (D + 31) / 32;              // 8-byte pieces: key group tid % 8 of channels tid / 8 + 32 i
    constexpr int MY_TILES = (DT + 3) / 4;                   // channel tiles of one wavefront: dt = wave + 4 i
    __shared__ __attribute__((aligned(16))) bf16 ks[2][32 * KROW];
    __shared__ __attribute__((aligned(16))) bf16 vs[2][D * VROW];
    __shared__ int pages[DECODE_LDS_PAGES];

    // the key/value heads of a token are neighbours in the grid: they start together and walk the same pages at the
    // same pace, so that the 4 KB pieces of a page that they read (one per head, next to each other) are asked for
    // at about the same time (steps of 96 to 256 requests 1 to 2 % shorter than with the tokens as neighbours)
    const int ti = blockIdx.y;
    const int t = token_list ? token_list[ti] : ti;
    const int G = nq / nkv, HB = (G + 15) / 16;
    const int kvh = blockIdx.x / HB, hb = blockIdx.x % HB;
    const int split = blockIdx.z;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;

    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* table = block_table + (int64_t)token_entry[t] * max_blocks;
    int begin, end;                                  // this split's keys, inclusive
    decode_split_range(p, lo, split, split_len, num_splits, begin, end);
    const int hloc = hb * 16 + r;
    const int head = kvh * G + (hloc < G ? hloc : G - 1);

    const float scale_log2 = scale * 1.44269504088896341f;
    float m_run = -INFINITY, l_run = 0.f;            // running maximum (in base-2 units) and sum
    f32x4 acc[MY_TILES];
#pragma unroll
    for (int i = 0; i < MY_TILES; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (begin <= end) {                                      // the whole workgroup takes the same branch
        const bf16* qrow = q + (int64_t)t * q_stride + (int64_t)head * D;
        bf16x8 qf[QK_STEPS];
#pragma unroll
        for (int c = 0; c < DT / 2; ++c) qf[c] = ld8(qrow + c * 32 + g * 8);
        if (DT & 1) qf[QK_STEPS - 1] = half_step(qrow + (DT - 1) * 16 + g * 4);

        const int vlo = begin & ~3, vhi = end & ~3;
        // The page size is a power of two here (the launcher sees to it): page arithmetic is shift and mask.
        // The split's pages (at most DECODE_LDS_PAGES, also the launcher's duty) are copied to LDS once, so
        // that a tile's addresses never wait for a read of the table from memory: such a wait would also wait
        // for every tile load issued before it.
        const int shift = __builtin_ctz(page_size);
        auto page_offset = [&](int pos) { return pos & (page_size - 1); };
        // The list covers the 32-key tiles whole (before the first visible key the table's own entries, past the
        // last one the last page again): every key of a tile has an address that may be read, and the keys
        // outside the split are masked.
        const int page_lo = (begin & ~31) >> shift, page_last = end >> shift;
        const int page_count = ((end | 31) >> shift) - page_lo + 1;
        for (int i = tid; i < page_count; i += 256) pages[i] = table[min(page_lo + i, page_last)];
        __syncthreads();
        auto page_of = [&](int pos) -> int64_t { return pages[(pos >> shift) - page_lo]; };
        const int64_t page_stride = (int64_t)nkv * page_size * D;      // elements from one page to the next
        const bf16* k_head = kc + (int64_t)kvh * page_size * D;
        const bf16* v_head = vc + (int64_t)kvh * page_size * D;
        // two register sets: the tiles two and three steps ahead are in flight while one is computed
        bf16x8 kreg_a[K_PER_THREAD], kreg_b[K_PER_THREAD];
        short4_t vreg_a[V_PER_THREAD], vreg_b[V_PER_THREAD];
        auto fetch = [&](bf16x8 (&kreg)[K_PER_THREAD], short4_t (&vreg)[V_PER_THREAD], int j0) {
#pragma unroll
            for (int i = 0; i < K_PER_THREAD; ++i) {
                const int c = tid + i * 256;
                if (K_CHUNKS % 256 == 0 || c < K_CHUNKS) {
                    const int row = c / (D / 8), col = c % (D / 8);
                    const int pos = j0 + row;
                    kreg[i] = ld8_once(k_head + page_of(pos) * page_stride + (page_offset(pos) * D + col * 8));
                }
            }
            const int kg = tid & 7;
            int vpos = j0 + kg * 4;
            vpos = vpos < vlo ? vlo : (vpos > vhi ? vhi : vpos);
            const bf16* vbase = v_head + page_of(vpos) * page_stride + page_offset(vpos);
#pragma unroll
            for (int i = 0; i < V_PER_THREAD; ++i) {
                const int d = (tid >> 3) + 32 * i;
                if (D % 32 == 0 || d < D) vreg[i] = ld4_once(vbase + (int64_t)d * page_size);
            }
            if (vpos == vlo || vpos == vhi) {          // the groups that hold the first and the last visible key
#pragma unroll
                for (int i = 0; i < V_PER_THREAD; ++i) vreg[i] = keep_visible(vreg[i], vpos, begin, end);
            }
        };
        auto stash = [&](const bf16x8 (&kreg)[K_PER_THREAD], const short4_t (&vreg)[V_PER_THREAD], int buf) {
#pragma unroll
            for (int i = 0; i < K_PER_THREAD; ++i) {
                const int c = tid + i * 256;
                if (K_CHUNKS % 256 == 0 || c < K_CHUNKS) {
                    const int row = c / (D / 8), col = c % (D / 8);
                    *reinterpret_cast<bf16x8*>(&ks[buf][row * KROW + col * 8]) = kreg[i];
                }
            }
            const int kg = tid & 7;
#pragma unroll
            for (int i = 0; i < V_PER_THREAD; ++i) {
                const int d = (tid >> 3) + 32 * i;
                if (D % 32 == 0 || d < D) *reinterpret_cast<short4_t*>(&vs[buf][d * VROW + kg * 4]) = vreg[i];
            }
        };
        auto compute = [&](int buf, int j0) {
            f32x4 s[2];
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const bf16* krow = &ks[buf][(half * 16 + r) * KROW];
                s[half] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < DT / 2; ++c)
                    s[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(krow + c * 32 + g * 8),
                                                                      qf[c], s[half], 0, 0, 0);
                if (DT & 1) {
                    union { bf16x8 wide; short4_t half4[2]; } u;
                    u.half4[0] = *reinterpret_cast<const short4_t*>(krow + (DT - 1) * 16 + g * 4);
                    u.half4[1] = short4_t{0, 0, 0, 0};
                    s[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u.wide, qf[QK_STEPS - 1], s[half], 0, 0, 0);
                }
            }
            // s[half][i] = S[key j0 + 16 half + 4 g + i][head r], still unscaled; keys outside the split are
            // masked (only the first and last step of a split can hold any)
            if (j0 < begin || j0 + 31 > end) {
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int key = j0 + half * 16 + g * 4 + i;
                        if (key < begin || key > end) s[half][i] = -INFINITY;
                    }
            }
            float mx = max3(max3(s[0][0], s[0][1], s[0][2]), max3(s[0][3], s[1][0], s[1][1]), max2(s[1][2], s[1][3]));
            mx = lanes4_max(mx) * scale_log2;                // scale > 0: the maximum commutes with it
            // running maximum and weights in base 2: weight = 2^(s * scale * log2(e) - m)
            const float m_new = max2(m_run, mx);             // finite: every 32-key step holds a visible key
            const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
            float pr[2][4], sum = 0.f;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    pr[half][i] = __builtin_amdgcn_exp2f(fmaf(s[half][i], scale_log2, -m_new));
                    sum += pr[half][i];
                }
            sum = lanes4_sum(sum);
            l_run = l_run * corr + sum;
            m_run = m_new;
            const bf16x8 pf = {(bf16)pr[0][0], (bf16)pr[0][1], (bf16)pr[0][2], (bf16)pr[0][3],
                               (bf16)pr[1][0], (bf16)pr[1][1], (bf16)pr[1][2], (bf16)pr[1][3]};
#pragma unroll
            for (int i = 0; i < MY_TILES; ++i) {
                const int dt = wave + 4 * i;
                if (DT % 4 == 0 || dt < DT) {
                    const bf16* vrow = &vs[buf][(dt * 16 + r) * VROW];
                    union { bf16x8 wide; short4_t half4[2]; } v;
                    v.half4[0] = *reinterpret_cast<const short4_t*>(vrow + g * 4);
                    v.half4[1] = *reinterpret_cast<const short4_t*>(vrow + 16 + g * 4);
                    acc[i] *= corr;
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v.wide, pf, acc[i], 0, 0, 0);
                }
            }
        };

        const int j_begin = begin & ~31;
        const int n = (end - j_begin) / 32 + 1;              // 32-key steps of this split
        // Every step stashes and fetches unconditionally (past the end: the last step once more, into a buffer
        // nobody reads), so the number of loads in flight at each wait is known when the kernel is compiled
        // and a wait for one register set does not also wait for the other.
        auto step_at = [&](int c) { return j_begin + 32 * (c < n ? c : n - 1); };
        fetch(kreg_a, vreg_a, j_begin);
        stash(kreg_a, vreg_a, 0);
        fetch(kreg_a, vreg_a, step_at(1));                   // odd steps travel in set a, even ones in set b
        fetch(kreg_b, vreg_b, step_at(2));
        __syncthreads();
        for (int c = 0; c < n; c += 2) {
            compute(0, j_begin + 32 * c);
            stash(kreg_a, vreg_a, 1);
            fetch(kreg_a, vreg_a, step_at(c + 3));
            __syncthreads();
            if (c + 1 >= n) break;
            compute(1, j_begin + 32 * (c + 1));
            stash(kreg_b, vreg_b, 0);
            fetch(kreg_b, vreg_b, step_at(c + 4));
            __syncthreads();
        }
    }

    // acc[i][j] = O^T[d = (wave + 4 i) * 16 + 4 g + j][head r]; every wavefront holds the same m_run, l_run
    const int hq = kvh * G + hloc;
    if (hloc < G) {
#pragma unroll
        for (int i = 0; i < MY_TILES; ++i) {
            const int dt = wave + 4 * i;
            if (DT % 4 == 0 || dt < DT) {
                const int d = dt * 16 + g * 4;
                if (num_splits == 1) {
                    const float inv = 1.0f / l_run;
                    bf16x4 o = {(bf16)(acc[i][0] * inv), (bf16)(acc[i][1] * inv), (bf16)(acc[i][2] * inv),
                                (bf16)(acc[i][3] * inv)};
                    *reinterpret_cast<bf16x4*>(out + ((int64_t)t * nq + hq) * D + d) = o;
                } else {
                    const int64_t slot = ((int64_t)ti * nq + hq) * num_splits + split;
                    *reinterpret_cast<f32x4*>(part_acc + slot * D + d) = acc[i];
                }
            }
        }
        if (num_splits > 1 && wave == 0 && g == 0) {
            const int64_t slot = ((int64_t)ti * nq + hq) * num_splits + split;
            part_ml[slot * 2] = m_run * 0.693147180559945309f;      // the merge works in natural units
            part_ml[slot * 2 + 1] = l_run;
        }
    }
}

// Merge the splits of one (token, head) in split order.  The weights exp(m_s - m) of the splits are
// computed once into LDS; then each thread sums one channel over the splits.
#define COMBINE_MAX_SPLITS 1024
__global__ void __launch_bounds__(128)
attention_combine_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                         const int* __restrict__ token_list, int nq, int D, int num_splits,
                         bf16* __restrict__ out) {
    __shared__ float factor[COMBINE_MAX_SPLITS];
    __shared__ float red[16];
    const int ti = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int t = token_list ? token_list[ti] : ti;
    const int64_t base = ((int64_t)ti * nq + h) * num_splits;
    float mx = -INFINITY;
    for (int s = tid; s < num_splits; s += 128)
        if (part_ml[(base + s) * 2 + 1] > 0.f) mx = fmaxf(mx, part_ml[(base + s) * 2]);
    const float m_all = block_max<128>(mx, red);
    float lsum = 0.f;
    for (int s = tid; s < num_splits; s += 128) {
        const float l = part_ml[(base + s) * 2 + 1];
        const float f = l > 0.f ? expf(part_ml[(base + s) * 2] - m_all) : 0.f;
        factor[s] = f;
        lsum += l * f;
    }
    const float l_all = block_sum<128>(lsum, red);      // also makes factor[] visible
    // every split wrote its partial output (zeros where it saw no key), so the loads need no condition and
    // are issued eight at a time
    for (int d = tid; d < D; d += 128) {
        const float* src = part_acc + base * D + d;
        float total = 0.f;
        int s = 0;
        for (; s + 8 <= num_splits; s += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[(int64_t)(s + u) * D];
#pragma unroll
            for (int u = 0; u < 8; ++u) total += v[u] * factor[s + u];
        }
        for (; s < num_splits; ++s) total += src[(int64_t)s * D] * factor[s];
        out[((int64_t)t * nq + h) * D + d] = (bf16)(total / l_all);
    }
}

// The longest range of keys (a multiple of 64) that one workgroup of the kernel that stages tiles through LDS takes
// for this page size: its list of pages is in LDS.  Longer splits run the slower kernel that keeps tiles in registers.
extern "C" int somi_attention_decode_lds_split(int page_size) {
    if (page_size <= 0) return 0;
    return (DECODE_LDS_PAGES - 2 - 8) * page_size / 64 * 64;
}

template <int DT>
static int launch_decode(const void* q, int64_t q_stride, const void* kc, const void* vc, const int* block_table,
                         int max_blocks, const int* token_list, const int* token_entry, const int* positions,
                         int n_list, int nq, int nkv, int page_size, int window, float scale, int split_len,
                         int num_splits, void* out, float* part_acc, float* part_ml, hipStream_t stream) {
    const int waves = DT <= 8 ? 4 : 2;
    const int G = nq / nkv, HB = (G + 15) / 16;
    const size_t smem = (size_t)(waves * DT * 256 + waves * 32) * sizeof(float);
    const bool pow2_pages = (page_size & (page_size - 1)) == 0;
    if (DT >= 2 && DT <= 8 && pow2_pages && n_list <= 65535 &&
        split_len / page_size + 2 + 8 <= DECODE_LDS_PAGES)                                        // + a tile's overhang
        // head sizes 32..128: keys and values staged through LDS (two tiles fit)
        hipLaunchKernelGGL((attention_decode_lds_kernel<(DT >= 2 && DT <= 8 ? DT : 2)>), dim3(nkv * HB, n_list, num_splits),
                           dim3(256), 0, stream, (const bf16*)q, q_stride, (const bf16*)kc, (const bf16*)vc, block_table,
                           max_blocks, token_list, token_entry, positions, nq, nkv, page_size, window, scale, split_len,
                           num_splits, (bf16*)out, part_acc, part_ml);
    else
        hipLaunchKernelGGL((attention_decode_kernel<DT>), dim3(n_list, nkv * HB, num_splits), dim3(waves * 64), smem,
                           stream, (const bf16*)q, q_stride, (const bf16*)kc, (const bf16*)vc, block_table, max_blocks,
                           token_list, token_entry, positions, nq, nkv, page_size, window, scale, split_len, num_splits,
                           (bf16*)out, part_acc, part_ml);
    SOMI_LAUNCH_CHECK("attention_decode");
    if (num_splits > 1) {
        hipLaunchKernelGGL(attention_combine_kernel, dim3(n_list, nq), dim3(128), 0, stream, part_acc, part_ml,
                           token_list, nq, DT * 16, num_splits, (bf16*)out);
        SOMI_LAUNCH_CHECK("attention_combine");
    }
    return 0;
}

// Attention of the listed tokens (token_list: [n_list] indices into the step's tokens, or null for tokens
// 0 .. n_list - 1) over their requests' pages.  bfloat16 only; head_dim a multiple of 16 up to 256;
// page_size a multiple of 4.  k_cache [pages, nkv, page_size, D], v_cache [pages, nkv, D, page_size].
// With num_splits > 1, part_acc holds n_list * nq * num_splits * D floats and part_ml
// n_list * nq * num_splits * 2 floats; split_len is a multiple of 16 and split_len * num_splits covers every
// listed token's position.
extern "C" int somi_attention_decode(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                                     const int* block_table, int max_blocks, const int* token_list,
                                     const int* token_entry, const int* positions, int n_list, int nq, int nkv, int D,
                                     int page_size, int window, float scale, int split_len, int num_splits, void* out,
                                     float* part_acc, float* part_ml, hipStream_t stream) {
    SOMI_REQUIRE(n_list >= 0 && nq > 0 && nkv > 0 && max_blocks > 0, "attention_decode: bad sizes");
    SOMI_REQUIRE(nq % nkv == 0, "attention_decode: num_q_heads (%d) must be divisible by num_kv_heads (%d)", nq, nkv);
    SOMI_REQUIRE(D % 16 == 0 && D >= 16 && D <= 256, "attention_decode: head_dim %d must be a multiple of 16 up to 256", D);
    SOMI_REQUIRE(page_size > 0 && page_size % 4 == 0, "attention_decode: page size %d must be a multiple of 4", page_size);
    SOMI_REQUIRE(window >= 0, "attention_decode: window must be >= 0");
    SOMI_REQUIRE(num_splits >= 1 && num_splits <= COMBINE_MAX_SPLITS && split_len > 0 && split_len % 16 == 0,
                 "attention_decode: bad split (len %d, count %d)", split_len, num_splits);
    SOMI_REQUIRE(num_splits == 1 || (part_acc && part_ml), "attention_decode: a workspace is needed for %d splits", num_splits);
    SOMI_REQUIRE((uintptr_t)q % 16 == 0 && (q_stride * 2) % 16 == 0 && (uintptr_t)k_cache % 16 == 0 &&
                 (uintptr_t)v_cache % 8 == 0, "attention_decode: q, k and v must be 16-byte aligned");
    const int G = nq / nkv, HB = (G + 15) / 16;
    SOMI_REQUIRE(nkv * HB <= 65535, "attention_decode: too many heads");
    if (n_list == 0) return 0;
#define SOMI_DECODE(DT)                                                                                              \
    case DT:                                                                                                         \
        return launch_decode<DT>(q, q_stride, k_cache, v_cache, block_table, max_blocks, token_list, token_entry,    \
                                 positions, n_list, nq, nkv, page_size, window, scale, split_len, num_splits, out,   \
                                 part_acc, part_ml, stream)
    switch (D / 16) {
        SOMI_DECODE(1); SOMI_DECODE(2); SOMI_DECODE(3); SOMI_DECODE(4); SOMI_DECODE(5); SOMI_DECODE(6);
        SOMI_DECODE(7); SOMI_DECODE(8); SOMI_DECODE(9); SOMI_DECODE(10); SOMI_DECODE(11); SOMI_DECODE(12);
        SOMI_DECODE(13); SOMI_DECODE(14); SOMI_DECODE(15); SOMI_DECODE(16);
    }
#undef SOMI_DECODE
    return somi_fail("attention_decode: unsupported head_dim %d", D);
}
