// Causal attention of prompt portions over the paged cache on 32 x 32 x 16 matrix tiles, for head sizes 64 and 128
// and pages of 8 keys or more (a power of two).  somi_attention_prefill takes this kernel where it applies and
// its older kernels elsewhere; the contract (arguments, masks, what a portion sees) is the same.
//
// Reference: somi_inference/models/qwen2.py:158-186 and the flash-style kernel
// somi_inference/core/flash_attention_triton.py:31-194 (query tiles against key tiles with a running maximum and
// sum, base-2 exponentials with the scale folded in).
//
// How it maps to gfx950:
//   * a wavefront owns 32 queries of one head; a workgroup has 8 wavefronts: 4 query blocks x 2 key splits (128
//     queries; the two halves of the wavefronts take the 32-key tiles of a 64-key step in turn and join their
//     results through LDS at the end) or 8 query blocks (256 queries).  Every key/value tile that comes from L2
//     serves 128 or 256 queries;
//   * tiles come by direct-to-LDS loads of 16 bytes a lane, one step ahead, into two stages.  A key row's 16-byte
//     pieces are permuted (piece c of row r at place c ^ swz(r)) so that the 16 lanes of a 16-byte LDS read fall
//     into different banks; the permutation is applied on the global side of the load.  Page addresses of key rows
//     are wavefront-uniform (scalar arithmetic); page ids are read from an LDS copy of the request's block table
//     one step before they are used;
//   * S^T = K . Q^T with the key rows fed in an order that swaps bits 2 and 3 of the row index: a lane's 16
//     scores are then two runs of 8 consecutive keys, which is the B-operand layout of the second product, so the
//     weights go from the first product to the second in registers, and a value fragment is one 16-byte read of
//     the page's transposed values;
//   * of the scale (times log2 e for base 2) the power of two goes into the query fragments once, exactly; the
//     rest, a factor in [1, 2), multiplies the float32 scores on their way into exp2, so no score is computed from
//     a rounded query; the running reference point enters the score product as its addend; the reference point
//     follows the maximum lazily (only when a score passes it by more than 2^8), so outputs are rarely rescaled;
//     the row sums come from one more matrix product with a fragment of ones;
//   * measured on this part, LDS reads and matrix instructions of a compute unit do not overlap well: a step's
//     time is close to the sum of both, so the fragment reads per product are what bounds the kernel (one
//     16-byte read a lane per matrix instruction).
// Measured on an MI355X (28/4 heads of 128): 2,048 tokens 60 us (the 16 x 16 kernel: 75), 8,192 tokens 523 us (663),
// 512 tokens after 3,584 cached ones 76 us (108).
#include "common.h"
#include "attention_prefill_tile.h"

#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;

#define TILE_GLOBAL __attribute__((address_space(1)))
#define TILE_LDS __attribute__((address_space(3)))
#define TILE_FENCE() __builtin_amdgcn_sched_barrier(0)
#define TILE_LAZY 8.0f       // base-2 units by which a score may pass the reference point before it moves

// Maxima of scores, which are never NaN (keys that must not be seen are -inf): the bare instructions.
__device__ __forceinline__ float tile_max2(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float tile_max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
// lanes l and l ^ 32 hold the two halves of a query's keys
__device__ __forceinline__ float tile_pair_max(float v) {
    u32x2 b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return tile_max2(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// D: head size (64 or 128).  QBLK query blocks of 32 per workgroup, KS key splits; QBLK * KS wavefronts.
template <int D, int QBLK, int KS>
__global__ void __launch_bounds__(QBLK * KS * 64, 2)
prefill_tile_kernel(const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ kc, const bf16* __restrict__ vc,
                    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ entry_start,
                    const int* __restrict__ entry_first_pos, const int* __restrict__ entry_len, int nq, int nkv,
                    int page_size, int window, float scale_pow2, float scale_rest, bf16* __restrict__ out) {
    constexpr int THREADS = QBLK * KS * 64;
    constexpr int CH = D / 8;                    // 16-byte pieces of a key row
    constexpr int KROW = D * 2;                  // bytes
    constexpr int K_BYTES = 32 * KROW, V_BYTES = D * 64, TILE = K_BYTES + V_BYTES;
    constexpr int STAGE = KS * TILE;
    constexpr int QG = QBLK * 32, STEP = 32 * KS;
    constexpr int KSTEPS = D / 16, DBLK = D / 32;
    constexpr int LOADERS = QBLK < K_BYTES / 1024 ? QBLK : K_BYTES / 1024;   // wavefronts that load one tile
    constexpr int K_INSTR = K_BYTES / 1024 / LOADERS, V_INSTR = V_BYTES / 1024 / LOADERS;
    constexpr int K_ROWS_PER_INSTR = 1024 / KROW; // 4 (D = 128) or 8 (D = 64)
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    int* pages = reinterpret_cast<int*>(smem + 2 * STAGE);

    const int h = blockIdx.x, e = blockIdx.y;
    const int kvh = h / (nq / nkv);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qb = wave % QBLK, ks = wave / QBLK;
    const int col = lane & 31, hf = lane >> 5;
    const int start = entry_start[e];
    const int len = entry_len != nullptr ? entry_len[e] : entry_start[e + 1] - start;
    const int group = gridDim.z - 1 - blockIdx.z;
    const int g0 = group * QG;
    if (g0 >= len) return;
    const int pos0 = entry_first_pos[e];
    const int* table = block_table + (int64_t)e * max_blocks;
    const int wg_valid = len - g0 < QG ? len - g0 : QG;
    const int wg_first = pos0 + g0, wg_last = pos0 + g0 + wg_valid - 1;
    const int lo = (window > 0 && wg_first - window + 1 > 0) ? wg_first - window + 1 : 0;

    const int shift = __builtin_ctz(page_size);
    const int j_begin = lo & ~(STEP - 1);
    const int page_lo = j_begin >> shift, page_last = wg_last >> shift;
    const int page_count = (((wg_last | (STEP - 1)) >> shift) - page_lo) + 1;
    for (int i = tid; i < page_count; i += THREADS) pages[i] = table[min(page_lo + i, page_last)];
    __syncthreads();
    const int64_t page_bytes = (int64_t)nkv * page_size * D * 2;       // bytes from one page to the next
    const char* k_head = reinterpret_cast<const char*>(kc) + (int64_t)kvh * page_size * D * 2;
    const char* v_head = reinterpret_cast<const char*>(vc) + (int64_t)kvh * page_size * D * 2;

    // ---- this lane's part in the loads of a tile (the wavefronts of a key split load its tile)
    const int lw = __builtin_amdgcn_readfirstlane(qb % LOADERS);        // which loader of the tile
    const bool loads = __builtin_amdgcn_readfirstlane(qb) < LOADERS;
    const int ks_s = __builtin_amdgcn_readfirstlane(ks);
    // keys: instruction i of this wavefront covers rows (lw * K_INSTR + i) * K_ROWS_PER_INSTR ..; a lane takes
    // the piece that belongs at its LDS place: row r, place c holds piece c ^ swz(r).  The rows of an
    // instruction lie in one page (pages of 8 keys or more), so the page's address is the wavefront's and a
    // lane adds its own 32-bit offset.
    const int k_lrow = lane / CH, k_place = lane % CH;
    unsigned koff[K_INSTR];
#pragma unroll
    for (int i = 0; i < K_INSTR; ++i) {
        const int row = (lw * K_INSTR + i) * K_ROWS_PER_INSTR + k_lrow;
        const int swz = CH == 16 ? (row & 15) : ((row >> 1) & 7);
        koff[i] = k_lrow * KROW + ((k_place ^ swz) << 4);
    }
    // values: instruction i covers channels (lw * V_INSTR + i) * 16 .. + 15, 64 bytes (32 keys) each; place c of
    // channel d holds piece c ^ ((d >> 2) & 3); a piece is 8 keys, which lie in one page
    const int v_ld = lane >> 2, v_place = lane & 3;
    const int v_piece = v_place ^ ((v_ld >> 2) & 3);      // (d >> 2) & 3 with d = 16 n + v_ld
    const int v_key = v_piece * 8;                        // first key of the piece within the tile
    const int64_t v_lane = (int64_t)(lw * V_INSTR * 16 + v_ld) * page_size * 2;
    const int64_t v_step = (int64_t)16 * page_size * 2;   // from one instruction's channels to the next's

    // page ids of the next tile to load: read from the list one step before they are used
    int kpage[K_INSTR], vpage;
    auto look_up = [&](int step_index) {
        if (!loads) return;
        const int j0 = j_begin + step_index * STEP + 32 * ks_s;
#pragma unroll
        for (int i = 0; i < K_INSTR; ++i)
            kpage[i] = pages[((j0 + (lw * K_INSTR + i) * K_ROWS_PER_INSTR) >> shift) - page_lo];
        vpage = pages[((j0 + v_key) >> shift) - page_lo];
    };
    auto issue = [&](int step_index, int stage) {
        if (!loads) return;
        const int j0 = j_begin + step_index * STEP + 32 * ks_s;
        char* kt = smem + stage * STAGE + ks_s * TILE;
        char* vt = kt + K_BYTES;
#pragma unroll
        for (int i = 0; i < K_INSTR; ++i) {
            const int row0 = (lw * K_INSTR + i) * K_ROWS_PER_INSTR;
            const int page = __builtin_amdgcn_readfirstlane(kpage[i]);
            const char* base = k_head + page * page_bytes + ((j0 + row0) & (page_size - 1)) * KROW;
            __builtin_amdgcn_global_load_lds((const TILE_GLOBAL void*)(base + koff[i]), (TILE_LDS void*)(kt + row0 * KROW), 16, 0, 0);
        }
        {
            const char* base = v_head + vpage * page_bytes + (((j0 + v_key) & (page_size - 1)) * 2 + v_lane);
#pragma unroll
            for (int i = 0; i < V_INSTR; ++i) {
                const int d0 = (lw * V_INSTR + i) * 16;
                __builtin_amdgcn_global_load_lds((const TILE_GLOBAL void*)(base + i * v_step), (TILE_LDS void*)(vt + d0 * 64), 16, 0, 0);
            }
        }
    };

    // ---- this wavefront's queries
    const int q0 = g0 + qb * 32;
    const bool active = q0 < len;
    const int nvalid = active ? (len - q0 < 32 ? len - q0 : 32) : 0;
    const int w_first = pos0 + q0, w_last = pos0 + q0 + nvalid - 1;
    const int w_lo = (window > 0 && w_first - window + 1 > 0) ? w_first - window + 1 : 0;
    int qi = q0 + col;
    qi = qi < len ? qi : len - 1;
    const int p = pos0 + qi;                              // this lane's query position
    const int p_first = window > 0 ? p - window + 1 : 0;
    bf16x8 qf[KSTEPS];
    {
        const bf16* qrow = q + (int64_t)(start + qi) * q_stride + (int64_t)h * D;
#pragma unroll
        for (int k = 0; k < KSTEPS; ++k) {
            // Of the scale (times log2 e, the change to base 2) only its power of two goes into the query, which
            // bfloat16 takes without rounding; the rest, a factor in [1, 2), multiplies the float32 scores.  So the
            // scores are those of the unscaled product, as in the kernels that scale after it.
            const bf16x8 raw = *reinterpret_cast<const bf16x8*>(qrow + k * 16 + hf * 8);
#pragma unroll
            for (int x = 0; x < 8; ++x) qf[k][x] = (bf16)((float)raw[x] * scale_pow2);
        }
    }
    // Scores, m_run and neg_m are in units of the product of the power-of-two-scaled query: exp2 takes them times
    // scale_rest.
    // m_run: what the weights are relative to (-inf: nothing seen yet); neg_m: its negative in every register, the
    // addend of the score product, so that scores arrive with the maximum already subtracted
    float m_run = -INFINITY;
    f32x16 acc[DBLK], acc_l, neg_m;                       // acc_l: every register holds the query's sum of weights
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        acc_l[r] = 0.f;
        neg_m[r] = 0.f;
    }
#pragma unroll
    for (int b = 0; b < DBLK; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[b][r] = 0.f;
    bf16x8 ones;
#pragma unroll
    for (int x = 0; x < 8; ++x) ones[x] = (bf16)1.0f;

    // the key row that this lane feeds as row `col` of the A operand: bits 2 and 3 of the index swapped, so
    // that a lane's scores of a 16-key step are 8 consecutive keys
    const int krow = (col & ~12) | ((col & 4) << 1) | ((col & 8) >> 1);
    const int kswz = CH == 16 ? (krow & 15) : ((krow >> 1) & 7);
    const int vswz = (col >> 2) & 3;                      // (d >> 2) & 3 with d = 32 b + col
    // LDS addresses of this lane's operand pieces within stage 0 (the stage's offset is an immediate)
    unsigned kaddr[KSTEPS], vaddr[2];
    const unsigned lds0 = (unsigned)(uintptr_t)(TILE_LDS char*)smem;
#pragma unroll
    for (int k = 0; k < KSTEPS; ++k) kaddr[k] = lds0 + ks_s * TILE + krow * KROW + (((2 * k + hf) ^ kswz) << 4);
#pragma unroll
    for (int t = 0; t < 2; ++t) vaddr[t] = lds0 + ks_s * TILE + K_BYTES + col * 64 + (((2 * t + hf) ^ vswz) << 4);
    // register r of a lane holds key j0 + 16 (r / 8) + 8 hf + r % 8: it is hidden from the lane's query when
    // 16 (r / 8) + r % 8 > p - j0 - 8 hf
    const int p_rel = p - 8 * hf;

    const int num_steps = (wg_last - j_begin) / STEP + 1;
    auto compute = [&](int s, auto stage_tag) {
        constexpr int ST = decltype(stage_tag)::value * STAGE;
        const int j0 = j_begin + s * STEP + 32 * ks_s;
        if (active && j0 <= w_last && j0 + 31 >= w_lo) {
            bf16x8 kf[KSTEPS];
#pragma unroll
            for (int k = 0; k < KSTEPS; ++k) kf[k] = *(const TILE_LDS bf16x8*)(kaddr[k] + ST);
            TILE_FENCE();
            f32x16 sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[0], qf[0], neg_m, 0, 0, 0);
#pragma unroll
            for (int k = 1; k < KSTEPS; ++k) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[k], qf[k], sc, 0, 0, 0);
            TILE_FENCE();
            // the values' reads are on their way while the weights are computed
            bf16x8 vf[DBLK][2];
#pragma unroll
            for (int b = 0; b < DBLK; ++b)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    vf[b][t] = *(const TILE_LDS bf16x8*)(vaddr[t] + (ST + b * 2048));
            TILE_FENCE();
            if (j0 + 31 > w_first) {
                const int lim = p_rel - j0;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (16 * (r >> 3) + (r & 7) > lim) sc[r] = -INFINITY;
            }
            if (window > 0) {
                const int first = p_first - j0 - 8 * hf;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (16 * (r >> 3) + (r & 7) < first) sc[r] = -INFINITY;
            }
            float mx = tile_max3(tile_max3(sc[0], sc[1], sc[2]), tile_max3(sc[3], sc[4], sc[5]), tile_max3(sc[6], sc[7], sc[8]));
            mx = tile_max3(mx, tile_max3(sc[9], sc[10], sc[11]), tile_max3(sc[12], sc[13], sc[14]));
            mx = tile_pair_max(tile_max2(mx, sc[15]));              // relative to m_run (to 0 while nothing was seen)
            // The reference point follows the scores only when they pass it by more than TILE_LAZY (in base-2 units):
            // weights may then exceed 1 (up to 2^TILE_LAZY), which float32 sums and bfloat16 weights hold as well, and
            // the sums and outputs are rescaled rarely.  A query's decision depends on its own scores only.
            const bool fresh = m_run == -INFINITY;
            const bool move = fresh ? mx > -INFINITY : mx * scale_rest > TILE_LAZY;
            if (__builtin_amdgcn_ballot_w64(move) != 0) {
                const float delta = move ? mx : 0.f;      // how far the reference point moves up
                const float corr = fresh ? 0.f : __builtin_amdgcn_exp2f(-delta * scale_rest);
                m_run = move ? (fresh ? mx : m_run + mx) : m_run;
#pragma unroll
                for (int b = 0; b < DBLK; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[b][r] *= corr;
                acc_l[0] *= corr;
                const float neg = m_run == -INFINITY ? 0.f : -m_run;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    sc[r] -= delta;
                    neg_m[r] = neg;
                }
            }
            float pr[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) pr[r] = __builtin_amdgcn_exp2f(sc[r] * scale_rest);
            bf16x8 pf[2];
#pragma unroll
            for (int t = 0; t < 2; ++t)
                pf[t] = bf16x8{(bf16)pr[8 * t], (bf16)pr[8 * t + 1], (bf16)pr[8 * t + 2], (bf16)pr[8 * t + 3],
                               (bf16)pr[8 * t + 4], (bf16)pr[8 * t + 5], (bf16)pr[8 * t + 6], (bf16)pr[8 * t + 7]};
            // values of keys outside what this wavefront may see are zeroed: 0 x NaN is NaN
            if (j0 + 31 > w_last || j0 < w_lo) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int key0 = j0 + 16 * t + 8 * hf;
#pragma unroll
                    for (int x = 0; x < 8; ++x)
                        if (key0 + x > w_last || key0 + x < w_lo) {
#pragma unroll
                            for (int b = 0; b < DBLK; ++b) vf[b][t][x] = (bf16)0.f;
                        }
                }
            }
            TILE_FENCE();
#pragma unroll
            for (int t = 0; t < 2; ++t) {
#pragma unroll
                for (int b = 0; b < DBLK; ++b) acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[b][t], pf[t], acc[b], 0, 0, 0);
                acc_l = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pf[t], acc_l, 0, 0, 0);
            }
        }
    };
    look_up(0);
    issue(0, 0);
    if (num_steps > 1) look_up(1);
    for (int s = 0; s < num_steps; s += 2) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (s + 1 < num_steps) issue(s + 1, 1);
        compute(s, std::integral_constant<int, 0>{});
        if (s + 2 < num_steps) look_up(s + 2);
        if (s + 1 >= num_steps) break;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (s + 2 < num_steps) issue(s + 2, 0);
        compute(s + 1, std::integral_constant<int, 1>{});
        if (s + 3 < num_steps) look_up(s + 3);
    }
    float l_run = acc_l[0];

    if constexpr (KS == 2) {
        // the wavefronts of the odd tiles hand maxima, sums and outputs to those of the even tiles
        __syncthreads();
        constexpr int ITEMS = DBLK * 16 + 2;
        float* hand = reinterpret_cast<float*>(smem) + qb * ITEMS * 64 + lane;
        if (ks == 1) {
#pragma unroll
            for (int b = 0; b < DBLK; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) hand[(b * 16 + r) * 64] = acc[b][r];
            hand[DBLK * 16 * 64] = m_run;
            hand[(DBLK * 16 + 1) * 64] = l_run;
        }
        __syncthreads();
        if (ks == 1) return;
        const float m_other = hand[DBLK * 16 * 64], l_other = hand[(DBLK * 16 + 1) * 64];
        const float m_new = tile_max2(m_run, m_other);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float mine = __builtin_amdgcn_exp2f((m_run - m_use) * scale_rest);
        const float theirs = __builtin_amdgcn_exp2f((m_other - m_use) * scale_rest);
        l_run = l_run * mine + l_other * theirs;
#pragma unroll
        for (int b = 0; b < DBLK; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[b][r] = acc[b][r] * mine + hand[(b * 16 + r) * 64] * theirs;
    }
    if (!active || q0 + col >= len) return;
    // register r of block b: channel 32 b + 8 (r / 4) + 4 hf + r % 4
    const float inv = 1.0f / l_run;
    bf16* orow = out + ((int64_t)(start + q0 + col) * nq + h) * D + 4 * hf;
#pragma unroll
    for (int b = 0; b < DBLK; ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const bf16x4 o = {(bf16)(acc[b][4 * g] * inv), (bf16)(acc[b][4 * g + 1] * inv),
                              (bf16)(acc[b][4 * g + 2] * inv), (bf16)(acc[b][4 * g + 3] * inv)};
            *reinterpret_cast<bf16x4*>(orow + 32 * b + 8 * g) = o;
        }
}

template <int D, int QBLK, int KS>
static int launch_tile(const void* q, int64_t q_stride, const void* kc, const void* vc, const int* block_table, int max_blocks,
                       const int* entry_start, const int* entry_first_pos, const int* entry_len, int n_entries,
                       int max_entry_len, int nq, int nkv, int page_size, int window, float scale, void* out,
                       hipStream_t stream) {
    const int lds = somi_prefill_tile_lds(D, QBLK, KS, max_blocks, page_size, window);
    static int lds_allowed[64];                  // per device: the largest dynamic LDS this kernel has been allowed so far
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return somi_fail("attention_prefill_tile: hipGetDevice failed");
    if (lds > lds_allowed[device]) {
        const hipError_t err = hipFuncSetAttribute((const void*)prefill_tile_kernel<D, QBLK, KS>,
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (err != hipSuccess) return somi_fail("attention_prefill_tile: %d bytes of LDS refused: %s", lds, hipGetErrorString(err));
        lds_allowed[device] = lds;
    }
    const dim3 grid(nq, n_entries, ceil_div(max_entry_len, QBLK * 32));
    // scale * log2(e) = 2^e * rest with rest in [1, 2)
    int exponent = 0;
    const float rest = 2.f * frexpf(scale * 1.44269504088896341f, &exponent);
    const float pow2 = ldexpf(1.f, exponent - 1);
    hipLaunchKernelGGL((prefill_tile_kernel<D, QBLK, KS>), grid, dim3(QBLK * KS * 64), lds, stream, (const bf16*)q, q_stride,
                       (const bf16*)kc, (const bf16*)vc, block_table, max_blocks, entry_start, entry_first_pos, entry_len,
                       nq, nkv, page_size, window, pow2, rest, (bf16*)out);
    SOMI_LAUNCH_CHECK("attention_prefill_tile");
    return 0;
}

// Dynamic LDS of a launch: two stages of tiles, the request's visible pages, and what the key splits hand over.
int somi_prefill_tile_lds(int D, int qblk, int ks, int max_blocks, int page_size, int window) {
    const int tile = 32 * D * 2 + D * 64;
    int entries = max_blocks + 64 / page_size + 2;
    if (window > 0) entries = min(entries, (window + qblk * 32 + 128) / page_size + 4);
    int lds = 2 * ks * tile + entries * 4;
    if (ks == 2) lds = max(lds, qblk * (D / 32 * 16 + 2) * 256);
    return lds;
}

// Whether the tile kernel takes these sizes at all (head size, page size, and a page list that fits LDS).
bool somi_prefill_tile_applies(int D, int page_size, int max_blocks, int window) {
    if (D != 64 && D != 128) return false;
    if (page_size < 8 || (page_size & (page_size - 1)) != 0) return false;
    return somi_prefill_tile_lds(D, 4, 2, max_blocks, page_size, window) <= SOMI_PREFILL_TILE_LDS_MAX &&
           somi_prefill_tile_lds(D, 8, 1, max_blocks, page_size, window) <= SOMI_PREFILL_TILE_LDS_MAX;
}

// wide: 256 queries a workgroup (long prompts); else 128 queries and two key splits.
int somi_prefill_tile(const void* q, int64_t q_stride, const void* kc, const void* vc, const int* block_table,
                      int max_blocks, const int* entry_start, const int* entry_first_pos, const int* entry_len,
                      int n_entries, int max_entry_len, bool wide, int nq, int nkv, int D, int page_size, int window,
                      float scale, void* out, hipStream_t stream) {
#define SOMI_TILE(DD, QB, KS_)                                                                                          \
    return launch_tile<DD, QB, KS_>(q, q_stride, kc, vc, block_table, max_blocks, entry_start, entry_first_pos, entry_len, \
                                    n_entries, max_entry_len, nq, nkv, page_size, window, scale, out, stream)
    if (D == 128 && wide) SOMI_TILE(128, 8, 1);
    if (D == 128) SOMI_TILE(128, 4, 2);
    if (D == 64 && wide) SOMI_TILE(64, 8, 1);
    if (D == 64) SOMI_TILE(64, 4, 2);
#undef SOMI_TILE
    return somi_fail("attention_prefill_tile: head size %d is not taken", D);
}
