// Causal attention of prompt portions over the paged cache, bfloat16, on the matrix cores.
//
// Reference: somi_inference/models/qwen2.py:158-186 (scores, causal mask, float32 softmax, weights . v;
// query head h reads key/value head h // (nq / nkv)) and the flash-style Triton kernel
// somi_inference/core/flash_attention_triton.py:31-194 (query tiles against key tiles with a running
// maximum and sum, base-2 exponentials with the scale folded in, :26, 119-120, 286).  The reference's
// kernel sees only the tokens of its own call on contiguous tensors; this one reads keys and values through
// the block table, so a portion attends to everything cached before it and to itself: the step's keys
// and values are written to their pages before the launch.
//
// A wavefront owns QB blocks of 16 consecutive query tokens of one (request portion, query head) and walks
// the keys 32 at a time:
//   S^T[key, query] = K[key, :] . Q^T        v_mfma_f32_16x16x32_bf16, K rows as the A operand (16 B loads)
//   online softmax per query (= per lane column) in float32, base 2
//   O^T[d, query] += V^T[d, key] . P^T       v_mfma_f32_16x16x32_bf16; the two 16-key halves of P^T leave the
//                                            first product in the B-operand layout, and V is stored transposed
//                                            inside a page, so a lane reads 2 x 4 consecutive keys of a channel
// Every key tile is used for all QB query blocks from registers.  Key tiles are aligned to absolute
// positions (multiples of 32), so a query's arithmetic does not depend on how the prompt was cut.
#include "common.h"
#include "attention_prefill_tile.h"

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

__device__ __forceinline__ bf16x8 pld8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ short4_t pld4(const bf16* p) { return *reinterpret_cast<const short4_t*>(p); }
__device__ __forceinline__ bf16x8 phalf(const bf16* p) {
    union { bf16x8 wide; short4_t half[2]; } u;
    u.half[0] = pld4(p);
    u.half[1] = short4_t{0, 0, 0, 0};
    return u.wide;
}
__device__ __forceinline__ bf16x8 pjoin(short4_t lo, short4_t hi) {
    union { bf16x8 wide; short4_t half[2]; } u;
    u.half[0] = lo;
    u.half[1] = hi;
    return u.wide;
}

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

// Maximum / sum over the four lane groups (lanes l, l ^ 16, l ^ 32, l ^ 48) with the row-swap instructions
// of gfx950: v_permlane16_swap exchanges odd 16-lane rows of one operand with even rows of the other,
// v_permlane32_swap the upper and lower halves; no LDS round trip.
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
__device__ __forceinline__ float group_max(float v) {
    u32x2 a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = max2(__uint_as_float(a[0]), __uint_as_float(a[1]));
    u32x2 b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return max2(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float group_sum(float v) {
    u32x2 a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    u32x2 b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

template <int DT, int QB>
__global__ void __launch_bounds__(256)
attention_prefill_kernel(const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ kc,
                         const bf16* __restrict__ vc, const int* __restrict__ block_table, int max_blocks,
                         const int* __restrict__ entry_start, const int* __restrict__ entry_first_pos, const int* __restrict__ entry_len, int nq,
                         int nkv, int page_size, int window, float scale_log2, bf16* __restrict__ out) {
    constexpr int D = DT * 16;
    constexpr int QK_STEPS = (DT + 1) / 2;
    constexpr int QW = QB * 16;                         // queries per wavefront
    const int e = blockIdx.y, h = blockIdx.z;
    const int kvh = h / (nq / nkv);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
    const int start = entry_start[e];
    const int len = entry_len != nullptr ? entry_len[e] : entry_start[e + 1] - start;
    const int q0 = (blockIdx.x * (blockDim.x >> 6) + wave) * QW;
    if (q0 >= len) return;                              // no workgroup barrier is used below
    const int pos0 = entry_first_pos[e];
    const int nvalid = len - q0 < QW ? len - q0 : QW;
    const int* table = block_table + (int64_t)e * max_blocks;

    // queries: column r of block qb is token start + q0 + 16 qb + r (past the portion's end: its last token,
    // computed again and not stored)
    bf16x8 qf[QB][QK_STEPS];
    int pcol[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        int qi = q0 + qb * 16 + r;
        qi = qi < len ? qi : len - 1;
        pcol[qb] = pos0 + qi;
        const bf16* qrow = q + (int64_t)(start + qi) * q_stride + (int64_t)h * D;
#pragma unroll
        for (int c = 0; c < DT / 2; ++c) qf[qb][c] = pld8(qrow + c * 32 + g * 8);
        if (DT & 1) qf[qb][QK_STEPS - 1] = phalf(qrow + (DT - 1) * 16 + g * 4);
    }
    const int p_first = pos0 + q0, p_last = pos0 + q0 + nvalid - 1;
    const int lo = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;

    float m_run[QB], l_run[QB];
    f32x4 acc[QB][DT];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[qb][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    const int vlo = lo & ~3, vhi = p_last & ~3;
    for (int j0 = lo & ~31; j0 <= p_last; j0 += 32) {
        // keys of the two 16-key halves: lane reads rows j0 + r and j0 + 16 + r (addresses kept inside the
        // visible range; what lies outside is masked below)
        bf16x8 kf[2][QK_STEPS];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            int pos = j0 + half * 16 + r;
            pos = pos < lo ? lo : (pos > p_last ? p_last : pos);
            const int64_t page = table[pos / page_size];
            const bf16* krow = kc + ((page * nkv + kvh) * page_size + pos % page_size) * (int64_t)D;
#pragma unroll
            for (int c = 0; c < DT / 2; ++c) kf[half][c] = pld8(krow + c * 32 + g * 8);
            if (DT & 1) kf[half][QK_STEPS - 1] = phalf(krow + (DT - 1) * 16 + g * 4);
        }
        // values: channel dt * 16 + r at keys j0 + 4 g .. + 3 and j0 + 16 + 4 g .. + 3
        bf16x8 vf[DT];
        {
            int va = j0 + g * 4, vb = j0 + 16 + g * 4;
            va = va < vlo ? vlo : (va > vhi ? vhi : va);
            vb = vb < vlo ? vlo : (vb > vhi ? vhi : vb);
            const int64_t pa = table[va / page_size], pb = table[vb / page_size];
            const bf16* vbase_a = vc + (pa * nkv + kvh) * (int64_t)D * page_size + va % page_size;
            const bf16* vbase_b = vc + (pb * nkv + kvh) * (int64_t)D * page_size + vb % page_size;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                short4_t a4 = pld4(vbase_a + (int64_t)(dt * 16 + r) * page_size);
                short4_t b4 = pld4(vbase_b + (int64_t)(dt * 16 + r) * page_size);
                if (va == vlo || va == vhi) a4 = keep_visible(a4, va, lo, p_last);     // the first and the last visible key's groups
                if (vb == vlo || vb == vhi) b4 = keep_visible(b4, vb, lo, p_last);
                vf[dt] = pjoin(a4, b4);
            }
        }
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            f32x4 s[2];
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                s[half] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < QK_STEPS; ++c)
                    s[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[half][c], qf[qb][c], s[half], 0, 0, 0);
            }
            // s[half][i] = S[key j0 + 16 half + 4 g + i][query column r of block qb]
            const int p = pcol[qb];
            const int first = window > 0 ? p - window + 1 : 0;
            float mx = -INFINITY;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = j0 + half * 16 + g * 4 + i;
                    s[half][i] = (key <= p && key >= first) ? s[half][i] * scale_log2 : -INFINITY;
                    mx = fmaxf(mx, s[half][i]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[qb], mx);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;     // nothing visible yet: weights stay 0
            const float corr = exp2f(m_run[qb] - m_use);
            float pr[2][4], sum = 0.f;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    pr[half][i] = exp2f(s[half][i] - m_use);
                    sum += pr[half][i];
                }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            l_run[qb] = l_run[qb] * corr + sum;
            m_run[qb] = m_new;
            const bf16x8 pf = {(bf16)pr[0][0], (bf16)pr[0][1], (bf16)pr[0][2], (bf16)pr[0][3],
                               (bf16)pr[1][0], (bf16)pr[1][1], (bf16)pr[1][2], (bf16)pr[1][3]};
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                acc[qb][dt] *= corr;
                acc[qb][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pf, acc[qb][dt], 0, 0, 0);
            }
        }
    }

    // acc[qb][dt][i] = O^T[d = dt * 16 + 4 g + i][query column r]
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const int qi = q0 + qb * 16 + r;
        if (qi >= len) continue;
        const float inv = 1.0f / l_run[qb];
        bf16* orow = out + ((int64_t)(start + qi) * nq + h) * D + g * 4;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const bf16x4 o = {(bf16)(acc[qb][dt][0] * inv), (bf16)(acc[qb][dt][1] * inv),
                              (bf16)(acc[qb][dt][2] * inv), (bf16)(acc[qb][dt][3] * inv)};
            *reinterpret_cast<bf16x4*>(orow + dt * 16) = o;
        }
    }
}

// The same computation with the key and value tiles staged through LDS: the four wavefronts of a
// workgroup own 4 x 32 consecutive queries of one (portion, head) and walk the keys together, 32 at a time.
// All 256 threads fetch the next tile from the pages into registers while the current one is being used
// from LDS, then store it into the other LDS buffer; one barrier per step.  Every key and value is read
// from L2/HBM once per 128 queries instead of once per wavefront.
//   K tile in LDS: [32 keys][D + 8] (rows padded by 16 bytes: the 16 rows a 16-byte read touches fall into
//   different banks); V tile: [D channels][32 + 4 keys] (a row is 18 dwords: the 16 channels that an 8-byte
//   read serves at once fall into different pairs of the 32 banks; with 20 dwords a row the counters showed
//   twice the conflicts).
#define PREFILL_LDS_TOTAL (96 * 1024)   // LDS of a workgroup, tiles (static) and page list (dynamic) together, that a launch may ask for
// The launch shapes go with the number of workgroups per compute unit, so their bounds are multiples of the device's
// units (the figures in brackets: on the 256 units of an MI355X, where they were measured at 28 query heads).
static int prefill_wide_groups(int units) { return units * 75 / 32; }        // [600] from this many 128-query groups on, workgroups take 128 queries, else 64 (448 groups 72 against 82 us with 64 queries, 672 groups 136 against 119)
static int prefill_wide_groups_cached(int units) { return units; }           // [256] the same where at least half of the keys were cached before the step
static int prefill_tile_wide_groups(int units) { return 3 * units / 2; }     // [384] from this many 256-query groups on the tile kernel takes 256 queries a workgroup (336 groups, 3,072 tokens: 118 us either way; 448 groups, 4,096 tokens: 166 against 183)
static int prefill_key_split_below(int units) { return 7 * units / 2; }      // [896] below this many 64-query workgroups two wavefronts share a query block's keys
                                                                             // (448 workgroups 29 against 33 us, 512 tokens after 3,584 cached 83 against 108; 896 workgroups the same; 1,120 workgroups 94 against 89)
// The launch shapes of the LDS kernel; a caller may ask for one (tests do, to reach each at small sizes).
#define PREFILL_SHAPE_AUTO 0
#define PREFILL_SHAPE_NARROW 1     // 64 queries a workgroup
#define PREFILL_SHAPE_SPLIT 2      // 64 queries, two wavefronts share a query block's keys
#define PREFILL_SHAPE_WIDE 3       // 128 queries
#define PREFILL_SHAPE_TILE 4       // the 32 x 32 tile kernel: 128 queries a workgroup, two key splits
#define PREFILL_SHAPE_TILE_WIDE 5  // the 32 x 32 tile kernel: 256 queries a workgroup
#define PREFILL_KEY_SPLIT_REACH 1024  // keys are shared only where the longest workgroup walks at least this many (32 tiles)
// KS = 2: twice the wavefronts; each query block is owned by KS of them, which take the 32-key tiles in turn
// (tile index modulo KS, by absolute position) and join their sums, maxima and outputs through LDS at the
// end.  The longest workgroup, which sets the time of a short prompt, has half as many steps to walk.
template <int DT, int QB, int KS>
__global__ void __launch_bounds__(256 * KS, 2 * KS)     // the second figure: wavefronts per SIMD to leave room for
attention_prefill_lds_kernel(const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ kc,
                             const bf16* __restrict__ vc, const int* __restrict__ block_table, int max_blocks,
                             const int* __restrict__ entry_start, const int* __restrict__ entry_first_pos, const int* __restrict__ entry_len, int nq,
                             int nkv, int page_size, int window, float scale_log2, bf16* __restrict__ out) {
    constexpr int D = DT * 16;
    constexpr int QK_STEPS = (DT + 1) / 2;
    constexpr int QW = QB * 16, WAVES = 4, QG = WAVES * QW;             // 64 or 128 queries per workgroup
    constexpr int KROW = D + 8, VROW = 32 + 4;                          // padded LDS rows, in elements
    constexpr int K_CHUNKS = 32 * D / 8;                                // 16-byte pieces of a key tile
    constexpr int K_PER_THREAD = (K_CHUNKS + 255) / 256;
    constexpr int V_PER_THREAD = (D + 31) / 32;                         // 8-byte pieces (4 keys of a channel): a
                                                                        // thread takes key group tid % 8 of
                                                                        // channels tid / 8 + 32 i
    constexpr int THREADS = 256 * KS, STEP = 32 * KS;                   // keys a step of the workgroup covers
    __shared__ __attribute__((aligned(16))) bf16 ks[2][KS][32 * KROW];
    __shared__ __attribute__((aligned(16))) bf16 vs[2][KS][D * VROW];
    extern __shared__ int pages[];                          // the launcher sizes it for the widest visible range

    // Workgroups are handed out in the order of blockIdx.x, then y, then z: heads vary fastest (the query
    // heads of one key/value head run side by side and share its tiles in L2) and the query groups go from
    // the latest, which see the most keys, to the earliest, so that the compute units fill up with long
    // workgroups first and the short ones land beside them.
    const int h = blockIdx.x, e = blockIdx.y;
    const int kvh = h / (nq / nkv);
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = (tid >> 6) & 3;                        // the query block of this wavefront
    const int kh = tid >> 8;                                // which of a step's KS tiles it computes and fetches
    const int tid256 = tid & 255;
    const int start = entry_start[e];
    const int len = entry_len != nullptr ? entry_len[e] : entry_start[e + 1] - start;
    const int group = gridDim.z - 1 - blockIdx.z;
    const int g0 = group * QG;
    if (g0 >= len) return;                                  // the whole workgroup leaves together
    const int pos0 = entry_first_pos[e];
    const int* table = block_table + (int64_t)e * max_blocks;
    const int wg_valid = len - g0 < QG ? len - g0 : QG;
    const int wg_first = pos0 + g0, wg_last = pos0 + g0 + wg_valid - 1;
    const int lo = (window > 0 && wg_first - window + 1 > 0) ? wg_first - window + 1 : 0;
    const int vlo = lo & ~3, vhi = wg_last & ~3;

    // The pages of the visible range go to LDS once, so that a tile's addresses do not wait for a
    // table read from memory before its own loads can start.
    // (power-of-two page size and a list that fits LDS: the launcher's duty.  A read of
    // the table from memory inside the loop would make every tile wait for all loads issued before it.)
    // The list covers the steps' tiles whole: before the first visible key the table's own entries (pages that
    // a window has released read as page 0), past the last one the last page again.  So every key of a tile
    // has an address that may be read, and keys outside the visible range need no clamp: their scores are
    // masked.
    const int shift = __builtin_ctz(page_size);
    const int page_lo = (lo & ~(STEP - 1)) >> shift, page_last = wg_last >> shift;
    const int page_count = (((wg_last | (STEP - 1)) >> shift) - page_lo) + 1;
    for (int i = tid; i < page_count; i += THREADS) pages[i] = table[min(page_lo + i, page_last)];
    __syncthreads();
    auto page_of = [&](int pos) -> int64_t { return pages[(pos >> shift) - page_lo]; };
    auto page_offset = [&](int pos) { return pos & (page_size - 1); };
    const int64_t page_stride = (int64_t)nkv * page_size * D;          // elements from one page to the next
    const bf16* k_head = kc + (int64_t)kvh * page_size * D;
    const bf16* v_head = vc + (int64_t)kvh * page_size * D;

    // this wavefront's queries
    const int q0 = g0 + wave * QW;
    const bool active = q0 < len;
    const int nvalid = active ? (len - q0 < QW ? len - q0 : QW) : 0;
    const int w_last = pos0 + q0 + nvalid - 1;
    bf16x8 qf[QB][QK_STEPS];
    int pcol[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        int qi = q0 + qb * 16 + r;
        qi = qi < len ? qi : len - 1;
        pcol[qb] = pos0 + qi;
        const bf16* qrow = q + (int64_t)(start + qi) * q_stride + (int64_t)h * D;
#pragma unroll
        for (int c = 0; c < DT / 2; ++c) qf[qb][c] = pld8(qrow + c * 32 + g * 8);
        if (DT & 1) qf[qb][QK_STEPS - 1] = phalf(qrow + (DT - 1) * 16 + g * 4);
    }
    float m_run[QB], l_run[QB];
    f32x4 acc[QB][DT];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[qb][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // staging registers of the next two tiles: a tile's loads are issued two steps before it is used, so that
    // their latency has two steps of arithmetic to hide behind
    bf16x8 kregs[2][K_PER_THREAD];
    short4_t vregs[2][V_PER_THREAD];
    auto fetch = [&](bf16x8 (&kreg)[K_PER_THREAD], short4_t (&vreg)[V_PER_THREAD], int j_step) {
        const int j0 = j_step + 32 * kh;                     // this thread's tile of the step
#pragma unroll
        for (int i = 0; i < K_PER_THREAD; ++i) {
            const int c = tid256 + i * 256;
            if (K_CHUNKS % 256 == 0 || c < K_CHUNKS) {
                const int row = c / (D / 8), col = c % (D / 8);
                const int pos = j0 + row;
                kreg[i] = pld8(k_head + page_of(pos) * page_stride + (page_offset(pos) * D + col * 8));
            }
        }
        {
            const int kg = tid256 & 7;
            int vpos = j0 + kg * 4;
            vpos = vpos < vlo ? vlo : (vpos > vhi ? vhi : vpos);
            const bf16* vbase = v_head + page_of(vpos) * page_stride + page_offset(vpos);
#pragma unroll
            for (int i = 0; i < V_PER_THREAD; ++i) {
                const int d = (tid256 >> 3) + 32 * i;
                if (D % 32 == 0 || d < D) vreg[i] = pld4(vbase + (int64_t)d * page_size);
            }
            if (vpos == vlo || vpos == vhi) {          // the groups that hold the first and the last visible key
#pragma unroll
                for (int i = 0; i < V_PER_THREAD; ++i) vreg[i] = keep_visible(vreg[i], vpos, lo, wg_last);
            }
        }
    };
    auto stash = [&](const bf16x8 (&kreg)[K_PER_THREAD], const short4_t (&vreg)[V_PER_THREAD], int buf) {
#pragma unroll
        for (int i = 0; i < K_PER_THREAD; ++i) {
            const int c = tid256 + i * 256;
            if (K_CHUNKS % 256 == 0 || c < K_CHUNKS) {
                const int row = c / (D / 8), col = c % (D / 8);
                *reinterpret_cast<bf16x8*>(&ks[buf][kh][row * KROW + col * 8]) = kreg[i];
            }
        }
        {
            const int kg = tid256 & 7;
#pragma unroll
            for (int i = 0; i < V_PER_THREAD; ++i) {
                const int d = (tid256 >> 3) + 32 * i;
                if (D % 32 == 0 || d < D) *reinterpret_cast<short4_t*>(&vs[buf][kh][d * VROW + kg * 4]) = vreg[i];
            }
        }
    };

    const int j_begin = lo & ~(STEP - 1);
    fetch(kregs[0], vregs[0], j_begin);
    if (j_begin + STEP <= wg_last) fetch(kregs[1], vregs[1], j_begin + STEP);
    stash(kregs[0], vregs[0], 0);
    __syncthreads();
    // one step: the tiles from j_step on are in LDS buffer `buf`, the next ones are on their way into register
    // set `next`, and the set that was stored last takes the loads of the tiles after those
    auto step = [&](int j_step, int buf, bf16x8 (&knext)[K_PER_THREAD], short4_t (&vnext)[V_PER_THREAD],
                    bf16x8 (&kfree)[K_PER_THREAD], short4_t (&vfree)[V_PER_THREAD]) {
        const bool more = j_step + STEP <= wg_last;
        if (j_step + 2 * STEP <= wg_last) fetch(kfree, vfree, j_step + 2 * STEP);
        const int j0 = j_step + 32 * kh;                     // this wavefront's tile of the step
        if (active && j0 <= w_last) {
            bf16x8 kf[2][QK_STEPS];
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const bf16* krow = &ks[buf][kh][(half * 16 + r) * KROW];
#pragma unroll
                for (int c = 0; c < DT / 2; ++c) kf[half][c] = *reinterpret_cast<const bf16x8*>(krow + c * 32 + g * 8);
                if (DT & 1) {
                    union { bf16x8 wide; short4_t half4[2]; } u;
                    u.half4[0] = *reinterpret_cast<const short4_t*>(krow + (DT - 1) * 16 + g * 4);
                    u.half4[1] = short4_t{0, 0, 0, 0};
                    kf[half][QK_STEPS - 1] = u.wide;
                }
            }
            // all query blocks stage by stage, so that their dependent chains overlap
            f32x4 s[QB][2];
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    s[qb][half] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int c = 0; c < QK_STEPS; ++c)
                        s[qb][half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[half][c], qf[qb][c], s[qb][half], 0, 0, 0);
                }
            // scores stay unscaled; keys a query must not see are masked, which only steps that reach past the
            // wavefront's first query (or a window's lower edge) can hold
            if (window > 0 || j0 + 31 > pos0 + q0) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) {
                    const int p = pcol[qb];
                    const int first = window > 0 ? p - window + 1 : 0;
#pragma unroll
                    for (int half = 0; half < 2; ++half)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int key = j0 + half * 16 + g * 4 + i;
                            if (key > p || key < first) s[qb][half][i] = -INFINITY;
                        }
                }
            }
            float mx[QB];
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
                mx[qb] = max3(max3(s[qb][0][0], s[qb][0][1], s[qb][0][2]), max3(s[qb][0][3], s[qb][1][0], s[qb][1][1]),
                              max2(s[qb][1][2], s[qb][1][3]));
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) mx[qb] = group_max(mx[qb]) * scale_log2;   // scale > 0 commutes with max
            float corr[QB], sum[QB];
            bf16x8 pf[QB];
            bool rescale = false;
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                const float m_new = max2(m_run[qb], mx[qb]);
                const float m_use = m_new == -INFINITY ? 0.f : m_new;     // nothing visible yet: weights stay 0
                corr[qb] = __builtin_amdgcn_exp2f(m_run[qb] - m_use);
                rescale = rescale || m_new != m_run[qb];
                m_run[qb] = m_new;
                float pr[2][4];
                sum[qb] = 0.f;
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        pr[half][i] = __builtin_amdgcn_exp2f(fmaf(s[qb][half][i], scale_log2, -m_use));
                        sum[qb] += pr[half][i];
                    }
                pf[qb] = bf16x8{(bf16)pr[0][0], (bf16)pr[0][1], (bf16)pr[0][2], (bf16)pr[0][3],
                                (bf16)pr[1][0], (bf16)pr[1][1], (bf16)pr[1][2], (bf16)pr[1][3]};
            }
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                sum[qb] = group_sum(sum[qb]);
                l_run[qb] = l_run[qb] * corr[qb] + sum[qb];
            }
            // the outputs are rescaled only when some query's maximum moved (rare after the first steps)
            if (__builtin_amdgcn_ballot_w64(rescale) != 0) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) acc[qb][dt] *= corr[qb];
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const bf16* vrow = &vs[buf][kh][(dt * 16 + r) * VROW];
                const bf16x8 vf = pjoin(*reinterpret_cast<const short4_t*>(vrow + g * 4),
                                        *reinterpret_cast<const short4_t*>(vrow + 16 + g * 4));
#pragma unroll
                for (int qb = 0; qb < QB; ++qb)
                    acc[qb][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[qb], acc[qb][dt], 0, 0, 0);
            }
        }
        if (more) stash(knext, vnext, buf ^ 1);
        __syncthreads();
    };
    for (int j0 = j_begin; j0 <= wg_last; j0 += 2 * STEP) {
        step(j0, 0, kregs[1], vregs[1], kregs[0], vregs[0]);
        if (j0 + STEP > wg_last) break;
        step(j0 + STEP, 1, kregs[0], vregs[0], kregs[1], vregs[1]);
    }

    if constexpr (KS == 2) {
        // the wavefronts of the odd tiles hand their maxima, sums and outputs to those of the even tiles (every
        // wavefront has passed the last step's barrier: the key tiles are done with)
        constexpr int ITEMS = QB * (DT * 4 + 2);
        float* hand = reinterpret_cast<float*>(&ks[0][0][0]) + wave * ITEMS * 64 + lane;
        static_assert(sizeof(ks) >= sizeof(float) * 4 * ITEMS * 64, "the key tiles hold what the wavefronts hand over");
        if (kh == 1) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                float* to = hand + qb * (DT * 4 + 2) * 64;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) to[(dt * 4 + i) * 64] = acc[qb][dt][i];
                to[DT * 4 * 64] = m_run[qb];
                to[(DT * 4 + 1) * 64] = l_run[qb];
            }
        }
        __syncthreads();
        if (kh == 1) return;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const float* from = hand + qb * (DT * 4 + 2) * 64;
            const float m_other = from[DT * 4 * 64], l_other = from[(DT * 4 + 1) * 64];
            const float m_new = max2(m_run[qb], m_other);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            const float mine = __builtin_amdgcn_exp2f(m_run[qb] - m_use), theirs = __builtin_amdgcn_exp2f(m_other - m_use);
            l_run[qb] = l_run[qb] * mine + l_other * theirs;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[qb][dt][i] = acc[qb][dt][i] * mine + from[(dt * 4 + i) * 64] * theirs;
        }
    }
    if (!active) return;
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const int qi = q0 + qb * 16 + r;
        if (qi >= len) continue;
        const float inv = 1.0f / l_run[qb];
        bf16* orow = out + ((int64_t)(start + qi) * nq + h) * D + g * 4;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const bf16x4 o = {(bf16)(acc[qb][dt][0] * inv), (bf16)(acc[qb][dt][1] * inv),
                              (bf16)(acc[qb][dt][2] * inv), (bf16)(acc[qb][dt][3] * inv)};
            *reinterpret_cast<bf16x4*>(orow + dt * 16) = o;
        }
    }
}

// Block-table entries a workgroup of the LDS kernel may list: the pages of its visible range (everything
// before its last query, or a window and the workgroup's 128 queries) and a 32-key tile's overhang.
// Static LDS of the LDS kernel: two buffers of KS key tiles [32][D + 8] and value tiles [D][36], bfloat16.
static int prefill_lds_static(int D, int ks) { return 2 * ks * (32 * (D + 8) + D * 36) * 2; }

static int prefill_page_entries(int max_blocks, int page_size, int window) {
    int entries = max_blocks + 16;                   // + the overhang of a step of two 32-key tiles, pages of 4 keys
    if (window > 0) entries = min(entries, (window + 128 + 128) / page_size + 16);
    return entries;
}

// The launch shape of the LDS kernel for a step.  128 queries per workgroup read every key and value tile half as
// often as 64 do, but the longest workgroup sets the time: with few workgroups the smaller ones spread better over
// the compute units.  Where most keys were cached before the step (max_context, the caller's hint of the longest
// context a portion ends at, is several portions long) all workgroups are long and the wide ones win earlier.  Few
// workgroups of 64 queries with many tiles each share a query block's keys between two wavefronts.
static int prefill_lds_choice(int n_entries, int max_entry_len, int max_context, int nq, int window, bool split_fits,
                              int units) {
    const int64_t wide_groups = (int64_t)ceil_div(max_entry_len, 128) * n_entries * nq;
    int reach = max_context;
    if (window > 0 && reach > window + max_entry_len) reach = window + max_entry_len;
    if (wide_groups >= prefill_wide_groups(units) ||
        (wide_groups >= prefill_wide_groups_cached(units) && reach >= 2 * max_entry_len))
        return PREFILL_SHAPE_WIDE;
    const int64_t narrow_groups = (int64_t)ceil_div(max_entry_len, 64) * n_entries * nq;
    if (narrow_groups < prefill_key_split_below(units) && reach >= PREFILL_KEY_SPLIT_REACH && split_fits)
        return PREFILL_SHAPE_SPLIT;
    return PREFILL_SHAPE_NARROW;
}

template <int DT>
static int launch_prefill_lds(const void* q, int64_t q_stride, const void* kc, const void* vc, const int* block_table,
                              int max_blocks, const int* entry_start, const int* entry_first_pos, const int* entry_len, int n_entries,
                              int max_entry_len, int max_context, int shape, int nq, int nkv, int page_size,
                              int window, float scale, void* out, hipStream_t stream) {
    const size_t page_list = (size_t)prefill_page_entries(max_blocks, page_size, window) * sizeof(int);
    const bool split_fits = (int)page_list + prefill_lds_static(DT * 16, 2) <= PREFILL_LDS_TOTAL;
    if (shape == PREFILL_SHAPE_AUTO)
        shape = prefill_lds_choice(n_entries, max_entry_len, max_context, nq, window, split_fits, somi_units());
    const bool wide = shape == PREFILL_SHAPE_WIDE;
    const dim3 grid(nq, n_entries, ceil_div(max_entry_len, wide ? 128 : 64));
    if (wide) {
        if (page_list > 16 * 1024)                       // with the tiles beyond the default limit of LDS
            (void)hipFuncSetAttribute((const void*)attention_prefill_lds_kernel<DT, 2, 1>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)page_list);
        hipLaunchKernelGGL((attention_prefill_lds_kernel<DT, 2, 1>), grid, dim3(256), page_list, stream, (const bf16*)q,
                           q_stride, (const bf16*)kc, (const bf16*)vc, block_table, max_blocks, entry_start,
                           entry_first_pos, entry_len, nq, nkv, page_size, window, scale * 1.44269504088896341f, (bf16*)out);
    } else if (shape == PREFILL_SHAPE_SPLIT && split_fits) {
        // few workgroups with many tiles each: the keys of a query block are split over two wavefronts
        if (page_list > 16 * 1024)
            (void)hipFuncSetAttribute((const void*)attention_prefill_lds_kernel<DT, 1, 2>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)page_list);
        hipLaunchKernelGGL((attention_prefill_lds_kernel<DT, 1, 2>), grid, dim3(512), page_list, stream, (const bf16*)q,
                           q_stride, (const bf16*)kc, (const bf16*)vc, block_table, max_blocks, entry_start,
                           entry_first_pos, entry_len, nq, nkv, page_size, window, scale * 1.44269504088896341f, (bf16*)out);
    } else {
        if (page_list > 16 * 1024)
            (void)hipFuncSetAttribute((const void*)attention_prefill_lds_kernel<DT, 1, 1>,
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)page_list);
        hipLaunchKernelGGL((attention_prefill_lds_kernel<DT, 1, 1>), grid, dim3(256), page_list, stream, (const bf16*)q,
                           q_stride, (const bf16*)kc, (const bf16*)vc, block_table, max_blocks, entry_start,
                           entry_first_pos, entry_len, nq, nkv, page_size, window, scale * 1.44269504088896341f, (bf16*)out);
    }
    SOMI_LAUNCH_CHECK("attention_prefill_lds");
    return 0;
}

template <int DT, int QB>
static int launch_prefill(const void* q, int64_t q_stride, const void* kc, const void* vc, const int* block_table,
                          int max_blocks, const int* entry_start, const int* entry_first_pos, const int* entry_len, int n_entries,
                          int max_entry_len, int nq, int nkv, int page_size, int window, float scale, void* out,
                          hipStream_t stream) {
    constexpr int WAVES = 4;
    const int per_group = WAVES * QB * 16;
    const dim3 grid(ceil_div(max_entry_len, per_group), n_entries, nq);
    hipLaunchKernelGGL((attention_prefill_kernel<DT, QB>), grid, dim3(WAVES * 64), 0, stream, (const bf16*)q, q_stride,
                       (const bf16*)kc, (const bf16*)vc, block_table, max_blocks, entry_start, entry_first_pos, entry_len, nq, nkv,
                       page_size, window, scale * 1.44269504088896341f, (bf16*)out);
    SOMI_LAUNCH_CHECK("attention_prefill");
    return 0;
}

// Attention of every token of every entry (portion) over its request's pages.  entry_start: [n_entries + 1]
// offsets of the portions in the flat token batch; entry_first_pos: [n_entries] position of each portion's
// first token; entry_len (or null): [n_entries] the portions' lengths where they differ from the offsets' (0 leaves a
// portion out: its tokens are somebody else's); max_entry_len: the longest portion (sizes the grid).  bfloat16 only; head_dim a multiple of 16
// up to 256; page_size a multiple of 4.  k_cache [pages, nkv, page_size, D], v_cache [pages, nkv, D, page_size];
// out: [n_tokens, nq * D].  max_context: the longest context a portion ends at (a hint for the launch shape; 0: unknown).
// shape: 0 lets the launcher choose; 1..3 ask for a launch shape of the 16 x 16 LDS kernel, 4 and 5 for one of the
// 32 x 32 tile kernel (PREFILL_SHAPE_*).
extern "C" int somi_attention_prefill(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                                      const int* block_table, int max_blocks, const int* entry_start,
                                      const int* entry_first_pos, const int* entry_len, int n_entries, int max_entry_len, int max_context,
                                      int shape, int nq, int nkv, int D, int page_size, int window, float scale,
                                      void* out, hipStream_t stream) {
    SOMI_REQUIRE(n_entries >= 0 && max_entry_len >= 0 && nq > 0 && nkv > 0 && max_blocks > 0,
                 "attention_prefill: bad sizes");
    SOMI_REQUIRE(nq % nkv == 0, "attention_prefill: num_q_heads (%d) must be divisible by num_kv_heads (%d)", nq, nkv);
    SOMI_REQUIRE(D % 16 == 0 && D >= 16 && D <= 256, "attention_prefill: head_dim %d must be a multiple of 16 up to 256", D);
    SOMI_REQUIRE(page_size > 0 && page_size % 4 == 0, "attention_prefill: page size %d must be a multiple of 4", page_size);
    SOMI_REQUIRE(window >= 0, "attention_prefill: window must be >= 0");
    SOMI_REQUIRE(scale >= 0.f, "attention_prefill: the scale of the scores must not be negative, got %g", (double)scale);
    SOMI_REQUIRE(shape >= PREFILL_SHAPE_AUTO && shape <= PREFILL_SHAPE_TILE_WIDE, "attention_prefill: unknown launch shape %d", shape);
    SOMI_REQUIRE(n_entries <= 65535 && nq <= 65535, "attention_prefill: too many entries or heads");
    SOMI_REQUIRE(max_entry_len <= 65535 * 128, "attention_prefill: a portion of %d tokens is too long", max_entry_len);
    SOMI_REQUIRE((uintptr_t)q % 16 == 0 && (q_stride * 2) % 16 == 0 && (uintptr_t)k_cache % 16 == 0 &&
                 (uintptr_t)v_cache % 8 == 0 && (uintptr_t)out % 8 == 0,
                 "attention_prefill: q, k, v and out must be 16-byte aligned");
    if (n_entries == 0 || max_entry_len == 0) return 0;
    // head sizes 64 and 128 over pages of 8 keys or more: the 32 x 32 tile kernel
    const bool tile_ok = somi_prefill_tile_applies(D, page_size, max_blocks, window) && (uintptr_t)v_cache % 16 == 0;
    if (shape >= PREFILL_SHAPE_TILE)
        SOMI_REQUIRE(tile_ok, "attention_prefill: the tile kernel does not take head size %d, pages of %d keys or a block table of %d pages",
                     D, page_size, max_blocks);
    if (tile_ok && (shape == PREFILL_SHAPE_AUTO || shape >= PREFILL_SHAPE_TILE)) {
        const int64_t groups = (int64_t)ceil_div(max_entry_len, 256) * n_entries * nq;
        const bool wide = shape == PREFILL_SHAPE_AUTO ? groups >= prefill_tile_wide_groups(somi_units()) : shape == PREFILL_SHAPE_TILE_WIDE;
        return somi_prefill_tile(q, q_stride, k_cache, v_cache, block_table, max_blocks, entry_start, entry_first_pos, entry_len,
                                 n_entries, max_entry_len, wide, nq, nkv, D, page_size, window, scale, out, stream);
    }
#define SOMI_PREFILL(DT, QB)                                                                                       \
    case DT:                                                                                                       \
        return launch_prefill<DT, QB>(q, q_stride, k_cache, v_cache, block_table, max_blocks, entry_start,         \
                                      entry_first_pos, entry_len, n_entries, max_entry_len, nq, nkv, page_size, window, scale, \
                                      out, stream)
#define SOMI_PREFILL_LDS(DT)                                                                                       \
    case DT:                                                                                                       \
        if (!lds_ok)                                                                                               \
            return launch_prefill<DT, 4>(q, q_stride, k_cache, v_cache, block_table, max_blocks, entry_start,      \
                                         entry_first_pos, entry_len, n_entries, max_entry_len, nq, nkv, page_size, window,    \
                                         scale, out, stream);                                                      \
        return launch_prefill_lds<DT>(q, q_stride, k_cache, v_cache, block_table, max_blocks, entry_start,         \
                                      entry_first_pos, entry_len, n_entries, max_entry_len, max_context, shape, nq, nkv,      \
                                      page_size, window, scale, out, stream)
    // head sizes 32..128 stage keys and values through LDS; the others (LDS would not hold two tiles, or a
    // tile is smaller than the workgroup's loads) keep them in registers per wavefront, and so do page sizes
    // that are no power of two and block tables too wide for the LDS copy of a request's pages
    const bool lds_ok = (page_size & (page_size - 1)) == 0 &&
                        prefill_page_entries(max_blocks, page_size, window) * 4 + prefill_lds_static(D, 1) <= PREFILL_LDS_TOTAL;
    switch (D / 16) {
        SOMI_PREFILL(1, 4); SOMI_PREFILL_LDS(2); SOMI_PREFILL_LDS(3); SOMI_PREFILL_LDS(4); SOMI_PREFILL_LDS(5);
        SOMI_PREFILL_LDS(6); SOMI_PREFILL_LDS(7); SOMI_PREFILL_LDS(8); SOMI_PREFILL(9, 2); SOMI_PREFILL(10, 2);
        SOMI_PREFILL(11, 2); SOMI_PREFILL(12, 2); SOMI_PREFILL(13, 2); SOMI_PREFILL(14, 2); SOMI_PREFILL(15, 2);
        SOMI_PREFILL(16, 2);
    }
#undef SOMI_PREFILL
#undef SOMI_PREFILL_LDS
    return somi_fail("attention_prefill: unsupported head_dim %d", D);
}

// The launch shape (PREFILL_SHAPE_*) that somi_attention_prefill chooses with shape 0 on a device of `units` compute
// units (0: the current device), given whether the tile kernel applies (head sizes 64 and 128, pages of 8 keys or
// more) and whether the LDS kernel's two-wavefront form fits LDS: what a test of the choice asks without a GPU.
extern "C" int somi_attention_prefill_choice(int n_entries, int max_entry_len, int max_context, int nq, int window,
                                             int tile_applies, int split_fits, int units) {
    if (units <= 0) units = somi_units();
    if (tile_applies) {
        const int64_t groups = (int64_t)ceil_div(max_entry_len, 256) * n_entries * nq;
        return groups >= prefill_tile_wide_groups(units) ? PREFILL_SHAPE_TILE_WIDE : PREFILL_SHAPE_TILE;
    }
    return prefill_lds_choice(n_entries, max_entry_len, max_context, nq, window, split_fits != 0, units);
}
