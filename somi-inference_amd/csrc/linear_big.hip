// Linear layer for many rows (prompt portions, decode batches beyond 64 requests):
// out[m, n] = sum_k x[m, k] * w[n, k], bfloat16 in, float32 accumulation on the matrix cores, with the
// feed-forward's and the block's element-wise work in the end of the product.
//
// Reference: the reference has a kernel of its own for the feed-forward's two products
// (somi_inference/core/mlp_triton.py:28-108, launched at :162-211, used at models/qwen2.py:231-249); its
// q/k/v and o products are nn.Linear (models/qwen2.py:268-271).  The forms here:
//   plain     out = s[m] * (x . w^T) + bias             (bfloat16; s: the row scale of an RMS norm, or 1)
//   swiglu    out = silu(s g) * (s u), g and u the gate and up products    (models/qwen2.py:226-229)
//   residual  h += x . w^T + bias in float32, in place (models/qwen2.py:333-339), leaving what the next
//             norm needs: bfloat16(norm_w * h) and the rows' sums of squares in partial sums; the same end
//             writes float32 results as they are (logits of many rows: somi_linear_big_f32).  Where the
//             tiles of this form are few (o and down of some hundred rows), the workgroups of a tile share
//             its K, each leaving its sums in a plane of a workspace, and a second kernel does the end.
//
// How it maps to gfx950:
//   * a workgroup owns a 256 x 256 or 256 x 128 tile of the output (128 x 256 for up to 128 rows) and walks K in stages of 64 (one
//     128-byte line per row: the L2 serves whole lines, half-used lines cost as much as full ones);
//   * both operands come by direct-to-LDS loads of 16 bytes a lane into a ring of stages (two for the wide
//     tile: 2 x 64 KB; three for the narrow one: 3 x 48 KB).  The 16-byte piece c of row r lies at piece
//     position c ^ ((r >> 1) & 7): the LDS has 64 banks of 4 bytes, so 16 lanes of a 16-byte read must
//     cover 256 distinct bytes; the permutation is applied on the global side of the load (a lane's LDS
//     position is fixed by the instruction);
//   * a wavefront computes 128 x 64 of the tile as 4 x 2 products of 32 x 32 x 16 (128 accumulator
//     registers); 8 wavefronts (wide) or 4 (narrow).  (The wide tile on four wavefronts of 128 x 128 each, their
//     sums in the accumulation registers, reads a third less from LDS per product and was measured slower:
//     2,048 x 37,888 x 3,584 in 521 us against 455, x 3,584 x 18,944 in 368 against 349; a wavefront's own LDS
//     reads do overlap its matrix instructions, but its waits at the barrier and for its loads leave the SIMD
//     with nothing to run, and the gated end of 128 x 128 sums spills.);
//   * fragment reads are software-pipelined one 16-deep sub-step ahead and issued between the products;
//     the order of instructions in the loop is pinned (the compiler's own schedule waited for each read
//     right after issuing it);
//   * products are taken transposed (D[n][m]): a lane then holds 4 consecutive columns of one row, so the
//     gate and up value of a channel (16 columns apart) meet in one lane, and a row's values are packed
//     and turned through LDS into stores of whole 128-byte rows;
//   * workgroups are numbered so that the eight dies (blockIdx % 8) each take a contiguous range of
//     tiles, the row tiles of one column tile next to each other: a weight tile is read from HBM by
//     one die only.
// Measured on an MI355X (2,048 rows): 256 x 128 tiles over K = 18,944 run at 1.2 PFLOP/s; 256 x 256 tiles
// over K = 3,584 and 37,888 columns at 1.2 (4.3 GB go from the L2s to the compute units per call; the products and
// the LDS reads alone take 370 to 386 us of the 455, five rounds of tiles for 4.6 rounds of work among them).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

#define BIG_GLOBAL __attribute__((address_space(1)))
#define BIG_LDS __attribute__((address_space(3)))
#define BIG_FENCE() __builtin_amdgcn_sched_barrier(0)

#define BIG_PLAIN 0
#define BIG_SWIGLU 1
#define BIG_RESIDUAL 2

#define BIG_BK 64                 // K per stage: one 128-byte line per row
#define BIG_ROW_BYTES 128
#define BIG_BM 256

// A stage's pieces past K read from here, so that a K that is no multiple of 64 adds zeros.
static __device__ __align__(16) unsigned int big_zero_piece[4];

struct BigArgs {
    const bf16* x; int64_t ldx;       // [M, K], row stride in elements
    const bf16* w; int64_t ldw;       // [N, K]
    const float* bias;                // [N] or null
    int M, N, K;
    int tiles_m, tiles_n;
    // plain / swiglu
    bf16* out;                        // [M, N] or [M, N / 2]
    int64_t ldo;                      // row stride of out in elements (a product over a range of columns writes into wider rows)
    const float* row_scale;           // [M] the rows' scales s, or null
    // residual
    float* h;                         // [M, N] float32, in and out
    int overwrite;                    // h is out only: h = x . w^T + bias (float32 results of many rows: logits)
    const float* norm_w;              // [N] or null
    bf16* weighted;                   // [M, N] = bfloat16(norm_w * h) or null
    float* stats_out;                 // [tiles_n * waves along n][stats_width] or null
    int stats_width;
    // residual with K split over workgroups (tiles of three whole stages only): each split leaves its sums in
    // partial [splits][M][N] and big_split_reduce_kernel does what the epilogue would have done
    float* partial;                   // or null: one workgroup walks the whole K
    int splits;                       // workgroups per tile: split s walks the stages s, s + splits, s + 2 splits, ...
                                      // (the splits of a tile run side by side and so read neighbouring lines of a row)
    int stats_rows;                   // rows of stats_out (one per 64 columns of the tiles)
    int reduce_plain;                 // the splits' sums end as the plain form does: out = s * sum + bias in bfloat16
                                      // (2: and are then rotated and stored, see big_split_reduce_rope_kernel; 3: they end as the
                                      // gated form does, see big_split_reduce_swiglu_kernel)
    // Streamed: the (tile, stage) units of the whole product, tiles in launch order, stages within a tile, are dealt
    // out to `stream_wgs` workgroups in equal contiguous ranges, so any number of tiles keeps every compute unit busy
    // to the end.  A range may begin or end inside a tile: such a segment leaves its sums in one of the workgroup's
    // two slots ([stream_wgs][2][BM x BN] float32: 0 for a segment that begins the range, 1 for one that ends it)
    // and big_stream_finish_kernel adds a tile's segments in stage order and does what the epilogue would have done.
    int stream_wgs;                   // 0: not streamed
    float* slots;
    // the q/k/v product whose splits' sums end rotated and stored (big_split_reduce_rope_kernel)
    const int* positions;             // [M]
    const int* cache_slots;           // [M]: page * page_size + offset of the token's k and v, or -1 for no store
    const float* inv_freq;            // [D / 2]
    bf16* k_cache;                    // [pages, nkv, page_size, D]
    bf16* v_cache;                    // [pages, nkv, D, page_size]
    int nq, nkv, D, page_size;
};

// silu(gate) * up = gate * up / (1 + e^-gate) with the hardware's base-2 exponential and reciprocal (each within
// one unit in the last place of float32; the result is rounded to bfloat16): nine instructions a value where expf and
// a float32 division take twenty-five, which a 2,048-row gate_up product feels (its end is 38.8 million values).
// The plain form's end, s * sum + bias, as one fused multiply-add in every kernel that computes it, so that a product
// gives the same bits whichever of them ends it (the compiler fuses the plain expression in some and not in others).
__device__ __forceinline__ float big_scale_bias(float scale, float sum, float bias) { return __builtin_fmaf(scale, sum, bias); }

__device__ __forceinline__ float big_silu_mul(float gate, float up) {
    return gate * up * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.44269504088896341f * gate));
}

template <int N> __device__ __forceinline__ void big_wait_vmcnt() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// One fragment read that the compiler does not track: every register it fills is named by the wait that
// precedes its first use (so that no use can be moved before the wait).
#define BIG_DS_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))

// S: 3 = a ring of three whole stages (narrow tile); 5 = five slots of 32 KB that hold one operand's stage each
// (wide tile), filled in the order A0 B0 A1 B1 A2 ...: piece q goes to slot q % 5.  While stage kt is computed,
// both pieces of stage kt + 1 are in the ring or on their way and A of kt + 2 is asked for; the barrier that ends the
// reads of stage kt frees two slots, which take B of kt + 2 at once and A of kt + 3 during stage kt + 1.  No
// wavefront asks for more than one load per product: every wavefront of a workgroup passes the barrier at the same
// time, and eight loads each in a burst filled the unit that takes their addresses, so that the wavefronts waited
// to issue and their matrix instructions with them (2,048 x 37,888 x 3,584: 526 us with the burst, 457 without).
// The wide form is persistent: a workgroup walks its die's tiles 32 apart, and the first pieces of the next
// tile are asked for before the finished tile is stored, so the stores and the first loads overlap.
// BM: rows of a tile, 256 (two wavefronts along m) or 128 (one: for 65 to 128 rows, where a 256-row tile would
// spend half of its products on rows that are not there).
// WONCE: the weight is read once (one row tile: every weight tile has a single reader), so its loads tell the caches
// not to keep the lines, as the few-rows products' weight streams do.
template <int BM, int BN, int S, int NW, int EPI, bool KTAIL, bool WONCE>
__global__ void __launch_bounds__(NW * 64, 1)
linear_big_kernel(const BigArgs p) {
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    constexpr int BK = BIG_BK, ROW_BYTES = BIG_ROW_BYTES;
    constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES, STAGE = A_BYTES + B_BYTES;
    constexpr int WAVES_M = BM / 128, WAVES_N = NW / WAVES_M;     // wavefronts along m and along n
    constexpr int WTM = 4, WTN = 2;                               // 32 x 32 products of a wavefront: 128 x 64
    static_assert(BM == WAVES_M * WTM * 32 && BN / WAVES_N == WTN * 32, "a wavefront owns 128 x 64 of the tile");
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW, L = LA + LB;  // direct loads a lane issues per stage (8 rows each)
    constexpr int KK = BK / 16, NM = WTM * WTN, NF = WTM + WTN;
    constexpr bool HALF = S == 5;
    static_assert(HALF || (S == 3 && L % KK == 0), "three whole stages, loads divisible over the sub-steps");
    static_assert(!HALF || (LA == LB && BN == 256 && BM == 256), "halves of equal size");
    constexpr int LPS = HALF ? 0 : L / KK;
    constexpr int SYNC_AFTER = 2;                                 // products of the last sub-step issued before the barrier
    constexpr int LSUB = HALF ? LA / KK : 1;                      // wide ring: loads of the far piece per sub-step
    static_assert(!HALF || (LA % KK == 0 && NM % LSUB == 0 && NM / LSUB > SYNC_AFTER && LA <= NF),
                  "the wide ring's loads spread over the sub-steps and the read slots");
    constexpr int HB = 256 * ROW_BYTES;                           // bytes of a slot of the wide ring
    constexpr int STG = HALF ? 3 * HB : 0;                        // where the epilogue stages: slots 3 and 4, or the ring
    constexpr int STG_WAVE = 8192;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int M = p.M, N = p.N, K = p.K;
    const bool streamed = p.stream_wgs > 0;
    const int splits = HALF || streamed ? 1 : p.splits;          // workgroups that share a tile's K
    const int KTF = (K + BK - 1) / BK;                            // stages of a whole tile
    int KT = KTF;                                                 // stages this workgroup walks: kt_first, kt_first + splits, ...
    int kt_first = 0;
    const int64_t stage_bytes = (int64_t)ROW_BYTES * splits;      // from one of its stages to the next
    const int lrow = lane >> 3, lpos = lane & 7;
    const int frow = lane & 31, fk = lane >> 5;
    const int ml = lane & 31, nh = lane >> 5;

    // tiles of this workgroup: the die (blockIdx % 8) owns a contiguous range of tiles with the row tiles of a
    // column tile next to each other; its workgroups take them 32 (wide, persistent) apart, or one each
    const int total = p.tiles_m * p.tiles_n * splits, per = (total + 7) / 8;
    const int die_first = (blockIdx.x & 7) * per, die_end = die_first + per < total ? die_first + per : total;
    const int stride = HALF ? (int)(gridDim.x >> 3) : per;
    int logical = die_first + (blockIdx.x >> 3);
    // streamed: the workgroups of a die hold neighbouring ranges of units (neighbouring tiles: what they share of
    // the operands meets in the die's L2); position pos owns the units [pos U / W, (pos + 1) U / W)
    const int pos = (blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3);
    int64_t unit = 0, unit_end = 0, unit_first = 0;
    if (streamed) {
        const int64_t units = (int64_t)p.tiles_m * p.tiles_n * KTF;
        unit_first = unit = units * pos / p.stream_wgs;
        unit_end = units * (pos + 1) / p.stream_wgs;
        if (unit >= unit_end) return;
    } else if (logical >= die_end) return;

    // ------------------------------------------------------------------ loads: global -> LDS
    // An instruction covers 8 rows of 128 bytes; lane l writes LDS position l % 8 of row l / 8 and reads the
    // global piece that belongs there.  Rows past the matrix repeat its last row (never stored).
    const char *xa, *wb;                       // first rows of the tile being loaded
    uint32_t offa[LA], offb[LB];
    int piece_a[LA], piece_b[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i) piece_a[i] = lpos ^ ((((wave * LA + i) * 8 + lrow) >> 1) & 7);
#pragma unroll
    for (int i = 0; i < LB; ++i) piece_b[i] = lpos ^ ((((wave * LB + i) * 8 + lrow) >> 1) & 7);
    // point the loads at a tile (and, with K split, at this split's stages; streamed: at the stages of the segment
    // that begins at unit `item`)
    auto aim = [&](int64_t item) {
        const int tile = streamed ? (int)(item / KTF) : (int)item / splits;
        const int tn = tile / p.tiles_m, tm = tile % p.tiles_m;
        const int mlim = M - tm * BM, nlim = N - tn * BN;
        xa = (const char*)(p.x + (int64_t)tm * BM * p.ldx);
        wb = (const char*)(p.w + (int64_t)tn * BN * p.ldw);
        if (streamed) {
            kt_first = (int)(item % KTF);
            const int64_t left = unit_end - item;
            KT = left < KTF - kt_first ? (int)left : KTF - kt_first;
            xa += (int64_t)kt_first * ROW_BYTES;
            wb += (int64_t)kt_first * ROW_BYTES;
        } else if (!HALF && splits > 1) {
            kt_first = (int)item % splits;
            KT = (KTF - kt_first + splits - 1) / splits;
            xa += (int64_t)kt_first * ROW_BYTES;
            wb += (int64_t)kt_first * ROW_BYTES;
        }
#pragma unroll
        for (int i = 0; i < LA; ++i) {
            const int row = (wave * LA + i) * 8 + lrow;
            offa[i] = (uint32_t)(row < mlim ? row : mlim - 1) * (uint32_t)p.ldx * 2u + (piece_a[i] << 4);
        }
#pragma unroll
        for (int i = 0; i < LB; ++i) {
            const int row = (wave * LB + i) * 8 + lrow;
            offb[i] = (uint32_t)(row < nlim ? row : nlim - 1) * (uint32_t)p.ldw * 2u + (piece_b[i] << 4);
        }
    };
    // load i of operand A (is_b false) or B of stage kt into LDS at byte offset `at`; a stage past the end repeats
    // the last one (it lands in a slot that is never read again)
    auto issue = [&](bool is_b, int kt, int at, int i) {
        kt = kt < KT ? kt : KT - 1;
        const char* src = (is_b ? wb + offb[i] : xa + offa[i]) + kt * stage_bytes;
        if (KTAIL) {
            if ((kt_first + kt * splits) * BK + (is_b ? piece_b[i] : piece_a[i]) * 8 >= K) src = (const char*)big_zero_piece;
        }
        char* dst = lds + at + (wave * (is_b ? LB : LA) + i) * 1024;
        if (WONCE && is_b) __builtin_amdgcn_global_load_lds((const BIG_GLOBAL void*)src, (BIG_LDS void*)dst, 16, 0, SOMI_LOAD_ONCE);
        else __builtin_amdgcn_global_load_lds((const BIG_GLOBAL void*)src, (BIG_LDS void*)dst, 16, 0, 0);
    };
    auto issue_piece = [&](int q, int slot, int i) { issue(q & 1, q >> 1, slot * HB, i); };                 // wide ring
    auto issue_stage = [&](int kt, int buf, int i) {                                                       // narrow ring
        if (i < LA) issue(false, kt, buf * STAGE, i); else issue(true, kt, buf * STAGE + A_BYTES, i - LA);
    };

    // ------------------------------------------------------------------ fragments: LDS -> registers
    const uint32_t lds_base = (uint32_t)(uintptr_t)(BIG_LDS char*)lds;
    uint32_t foffa[KK], foffb[KK];              // relative to the start of the operand's stage
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        const uint32_t f = frow * ROW_BYTES + (((kk * 2 + fk) ^ ((frow >> 1) & 7)) << 4);
        foffa[kk] = lds_base + f + wm * 128 * ROW_BYTES;
        foffb[kk] = lds_base + f + wn * (BN / WAVES_N) * ROW_BYTES;
    }
    // read q of a set, in the order the products need them: a[0], every b, then the other a
    auto read_one = [&](bf16x8 (&a)[WTM], bf16x8 (&b)[WTN], uint32_t aa, uint32_t ab, int q) {
        if (q == 0) BIG_DS_READ(a[0], aa, 0);
        else if (q == 1) BIG_DS_READ(b[0], ab, 0);
        else if (q == 2) BIG_DS_READ(b[1], ab, 32 * ROW_BYTES);
        else if (q == 3) BIG_DS_READ(a[1], aa, 32 * ROW_BYTES);
        else if (q == 4) BIG_DS_READ(a[2], aa, 64 * ROW_BYTES);
        else if (q == 5) BIG_DS_READ(a[3], aa, 96 * ROW_BYTES);
    };
    auto wait_frags = [&](bf16x8 (&a)[WTM], bf16x8 (&b)[WTN]) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]));
    };

    // the first tile's first pieces
    aim(streamed ? unit : (int64_t)logical);
    if (HALF) {
#pragma unroll
        for (int q = 0; q < 5; ++q)
#pragma unroll
            for (int i = 0; i < LA; ++i) issue_piece(q, q, i);
    } else {
#pragma unroll
        for (int st = 0; st < S - 1; ++st)
#pragma unroll
            for (int i = 0; i < L; ++i) issue_stage(st, st, i);
    }

    while (true) {
        const int tile = streamed ? (int)(unit / KTF) : logical / splits;
        const int tn = tile / p.tiles_m, tm = tile % p.tiles_m;
        const int m0 = tm * BM, n0 = tn * BN;
        const int next = logical + stride;
        // streamed: the segment [unit, unit + KT) of this tile; one that is not the tile's whole K goes to a slot
        const int64_t next_unit = unit + KT;
        const bool whole = !streamed || KT == KTF;
        float* const slot = streamed ? p.slots + ((int64_t)pos * 2 + (unit == unit_first ? 0 : 1)) * (BM * BN) : nullptr;
        const bool has_next = streamed ? next_unit < unit_end : HALF && next < die_end;

        f32x16 acc[WTM][WTN];
#pragma unroll
        for (int i = 0; i < WTM; ++i)
#pragma unroll
            for (int j = 0; j < WTN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        auto product = [&](bf16x8 (&a)[WTM], bf16x8 (&b)[WTN], int q) {
            const int i = q / WTN, j = q % WTN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);    // D[n][m]
        };
        bf16x8 a0[WTM], b0[WTN], a1[WTM], b1[WTN];

        // ---------------------------------------------------------------- the loop over K
        if constexpr (HALF) {
            big_wait_vmcnt<3 * LA>();          // pieces 0 and 1 have landed
            __syncthreads();
#pragma unroll
            for (int q = 0; q < NF; ++q) read_one(a0, b0, foffa[0], foffb[0] + HB, q);
            int sa = 0, sb = 1;                // slots of the stage computed on
            for (int kt = 0; kt < KT; ++kt) {
                const int na = sa + 2 >= 5 ? sa - 3 : sa + 2, nb = sb + 2 >= 5 ? sb - 3 : sb + 2;     // slots of the next stage
                const int sp = sa == 0 ? 4 : sa - 1;                                                   // the slot B of kt - 1 had
                BIG_FENCE();
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) {
                    const bool last = kk == KK - 1;
                    const uint32_t aa = last ? foffa[0] + na * HB : foffa[kk + 1 < KK ? kk + 1 : 0] + sa * HB;
                    const uint32_t ab = last ? foffb[0] + nb * HB : foffb[kk + 1 < KK ? kk + 1 : 0] + sb * HB;
                    BIG_FENCE();
                    if (kk & 1) wait_frags(a1, b1); else wait_frags(a0, b0);
                    BIG_FENCE();
                    int reads = 0, loads = 0;
#pragma unroll
                    for (int q = 0; q < NM; ++q) {
                        if (last && q == SYNC_AFTER) {
                            // stage kt + 1 has landed (only what this iteration has asked for of A of kt + 2 may still be
                            // on its way); everybody has read stage kt
                            big_wait_vmcnt<(KK - 1) * LSUB + 1>();
                            __builtin_amdgcn_s_barrier();
                            BIG_FENCE();
                        }
                        if (kk & 1) product(a1, b1, q); else product(a0, b0, q);
                        BIG_FENCE();
                        // A of stage kt + 2 (piece 2 kt + 4) into the slot that B of kt - 1 had: over the sub-steps
                        if (q % (NM / LSUB) == 0) {
                            issue_piece(2 * kt + 4, sp, kk * LSUB + q / (NM / LSUB));
                            BIG_FENCE();
                        }
                        if ((!last || q >= SYNC_AFTER) && reads < NF) {
                            if (kk & 1) read_one(a0, b0, aa, ab, reads); else read_one(a1, b1, aa, ab, reads);
                            ++reads;
                            // B of stage kt + 2 into the slot A of kt had, which the barrier has just freed
                            if (last && loads < LA) { issue_piece(2 * kt + 5, sa, loads); ++loads; }
                            BIG_FENCE();
                        }
                    }
                }
                sa = na;
                sb = nb;
            }
        } else {
            // three whole stages: the slot freed one iteration ago is refilled evenly over the sub-steps
            big_wait_vmcnt<(S - 2) * L>();
            __syncthreads();
#pragma unroll
            for (int q = 0; q < NF; ++q) read_one(a0, b0, foffa[0], foffb[0] + A_BYTES, q);
            int buf = 0, rbuf = S - 1;          // the stage computed on; the slot being refilled
            for (int kt = 0; kt < KT; ++kt) {
                const int nbuf = buf + 1 == S ? 0 : buf + 1;
                BIG_FENCE();
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) {
                    const bool last = kk == KK - 1;
                    const uint32_t aa = last ? foffa[0] + nbuf * STAGE : foffa[kk + 1 < KK ? kk + 1 : 0] + buf * STAGE;
                    const uint32_t ab = (last ? foffb[0] + nbuf * STAGE : foffb[kk + 1 < KK ? kk + 1 : 0] + buf * STAGE) + A_BYTES;
                    BIG_FENCE();
                    if (kk & 1) wait_frags(a1, b1); else wait_frags(a0, b0);
                    BIG_FENCE();
                    int reads = 0, loads = 0;
#pragma unroll
                    for (int q = 0; q < NM; ++q) {
                        if (last && q == SYNC_AFTER) {
                            // the next stage has landed and everybody has read this one
                            big_wait_vmcnt<(S - 3) * L + LPS * (KK - 1)>();
                            __builtin_amdgcn_s_barrier();
                            BIG_FENCE();
                        }
                        if (kk & 1) product(a1, b1, q); else product(a0, b0, q);
                        BIG_FENCE();
                        if ((!last || q >= SYNC_AFTER) && reads < NF) {
                            if (kk & 1) read_one(a0, b0, aa, ab, reads); else read_one(a1, b1, aa, ab, reads);
                            ++reads;
                            if (loads < LPS) { issue_stage(kt + S - 1, rbuf, kk * LPS + loads); ++loads; }
                            BIG_FENCE();
                        }
                    }
                }
                rbuf = buf;
                buf = nbuf;
            }
        }
        // every load of this tile has landed, every wavefront is done with the ring
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        // what the epilogue reads beside the sums, asked for before the next tile's loads: loads return in order,
        // so these must not queue behind them
        const int wave_n0 = n0 + wn * (BN / WAVES_N);            // first column of the wavefront
        float scale[WTM];
        float bv[WTN][EPI == BIG_PLAIN ? 16 : 1];
        if (EPI != BIG_RESIDUAL) {
#pragma unroll
            for (int i = 0; i < WTM; ++i) {
                const int sm = m0 + wm * 128 + i * 32 + ml;
                scale[i] = p.row_scale != nullptr ? p.row_scale[sm < M ? sm : M - 1] : 1.f;
            }
            if (EPI == BIG_PLAIN) {
#pragma unroll
                for (int j = 0; j < WTN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int gn = wave_n0 + j * 32 + 8 * (r >> 2) + 4 * nh + (r & 3);
                        bv[j][r] = p.bias != nullptr ? p.bias[gn < N ? gn : N - 1] : 0.f;
                    }
            }
        }
        if (HALF && has_next) {
            // the next tile's pieces A0 B0 A1 go out now, into the slots the stores below do not use
            aim(streamed ? next_unit : (int64_t)next);
#pragma unroll
            for (int q = 0; q < 3; ++q)
#pragma unroll
                for (int i = 0; i < LA; ++i) issue_piece(q, q, i);
        }

        // ---------------------------------------------------------------- epilogue
        // A product holds D[n][m]: lane l has row m = l % 32 and, in registers 4 g .. 4 g + 3, the columns
        // 8 g + 4 (l / 32) + 0..3 of its 32.  A wavefront turns 32 rows at a time through its own 8 KB of LDS
        // into whole rows and stores 16 bytes a lane.
        char* stg = lds + STG + wave * STG_WAVE;

        if (!whole) {
            // a segment of the tile's K: the sums as they are, whole rows of the tile-local slot
            constexpr int SROW = 32 * 4 + 16;
#pragma unroll
            for (int i = 0; i < WTM; ++i) {
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x16& t = acc[i][j];
                        f32x4 v = {t[4 * g], t[4 * g + 1], t[4 * g + 2], t[4 * g + 3]};
                        *(f32x4*)(stg + ml * SROW + (8 * g + 4 * nh) * 4) = v;
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                    for (int pass = 0; pass < 4; ++pass) {
                        const int row = pass * 8 + (lane >> 3), piece = lane & 7;
                        const f32x4 v = *(const f32x4*)(stg + row * SROW + piece * 16);
                        const int rt = wm * 128 + i * 32 + row, ct = wn * (BN / WAVES_N) + j * 32 + piece * 4;
                        *(f32x4*)(slot + rt * BN + ct) = v;
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                }
            }
        } else if (EPI == BIG_PLAIN || EPI == BIG_SWIGLU) {
            constexpr int CW = EPI == BIG_SWIGLU ? WTN * 16 : WTN * 32;      // output columns of the wavefront per row
            constexpr int SROW = CW * 2 + 8;                                   // staged row: 8 bytes of padding spread the banks
            constexpr int LPR = CW * 2 / 16;                                   // lanes per row when reading back
            const int out_n = EPI == BIG_SWIGLU ? N / 2 : N;
            const int out_c0 = EPI == BIG_SWIGLU ? wave_n0 / 2 : wave_n0;
            const bool aligned = (out_n & 7) == 0 && (p.ldo & 7) == 0 && ((uintptr_t)p.out & 15) == 0;
#pragma unroll
            for (int i = 0; i < WTM; ++i) {
                const float s = scale[i];            // the row scale of the norm whose rows x holds
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
                    const f32x16& t = acc[i][j];
                    if (EPI == BIG_SWIGLU) {
                        // registers r and r + 8 are gate and up of one channel (columns 16 apart)
#pragma unroll
                        for (int g = 0; g < 2; ++g) {
                            bf16x4 v;
#pragma unroll
                            for (int c = 0; c < 4; ++c) {
                                const float gate = s * t[4 * g + c], up = s * t[4 * g + c + 8];
                                v[c] = (bf16)big_silu_mul(gate, up);
                            }
                            *(bf16x4*)(stg + ml * SROW + (j * 16 + 8 * g + 4 * nh) * 2) = v;
                        }
                    } else {
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            bf16x4 v;
#pragma unroll
                            for (int c = 0; c < 4; ++c) v[c] = (bf16)big_scale_bias(s, t[4 * g + c], bv[j][4 * g + c]);
                            *(bf16x4*)(stg + ml * SROW + (j * 32 + 8 * g + 4 * nh) * 2) = v;
                        }
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                for (int pass = 0; pass < 32 * LPR / 64; ++pass) {
                    const int row = pass * (64 / LPR) + lane / LPR, piece = lane % LPR;
                    const u32x4 v = *(const u32x4*)(stg + row * SROW + piece * 16);
                    const int gm = m0 + wm * 128 + i * 32 + row;
                    const int gc = out_c0 + piece * 8;
                    if (gm < M) {
                        bf16* dst = p.out + (int64_t)gm * p.ldo + gc;
                        if (aligned && gc + 8 <= out_n) *(u32x4*)dst = v;
                        else {
                            const bf16* e = (const bf16*)&v;
                            for (int c = 0; c < 8; ++c)
                                if (gc + c < out_n) dst[c] = e[c];
                        }
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            }
        } else {
            // h += product (+ bias): 32 rows x 32 columns of float32 at a time; a row is read back by 8 lanes
            constexpr int SROW = 32 * 4 + 16;
            const bool aligned = (N & 3) == 0 && ((uintptr_t)p.h & 15) == 0 &&
                                 (p.weighted == nullptr || ((uintptr_t)p.weighted & 7) == 0);
            const int stats_row = tn * WAVES_N + wn;
            // With four wavefronts (512 registers each) the stream's values are asked for ahead of their use, a block
            // of 32 rows at a time (eight loads of 16 bytes a lane), the next block's while this one is added: a load
            // that is asked for where it is used waits for memory 32 times a tile (2,048 x 3,584 x 64, where the end
            // is all there is: 29 us, of which the stream's 73 MB would take 12).  The tile of eight wavefronts has no
            // registers to spare for it.
            constexpr bool DEEP = NW == 4;
            const bool ahead = DEEP && (HALF || p.partial == nullptr) && aligned && !p.overwrite;
            f32x4 hq[DEEP ? 2 : 1][WTN][4];
            auto ask = [&](int i, f32x4 (&q)[WTN][4]) {
#pragma unroll
                for (int j = 0; j < WTN; ++j)
#pragma unroll
                    for (int pass = 0; pass < 4; ++pass) {
                        const int gm = m0 + wm * 128 + i * 32 + pass * 8 + (lane >> 3);
                        const int gn = wave_n0 + j * 32 + (lane & 7) * 4;
                        q[j][pass] = gm < M && gn + 4 <= N ? *(const f32x4*)(p.h + (int64_t)gm * N + gn) : f32x4{0.f, 0.f, 0.f, 0.f};
                    }
            };
            if (ahead) ask(0, hq[0]);
#pragma unroll
            for (int i = 0; i < WTM; ++i) {
                float sq[4] = {0.f, 0.f, 0.f, 0.f};            // of the rows this lane reads back, over both products
                if (ahead && i + 1 < WTM) ask(i + 1, hq[DEEP ? (i + 1) & 1 : 0]);
#pragma unroll
                for (int j = 0; j < WTN; ++j) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x16& t = acc[i][j];
                        f32x4 v = {t[4 * g], t[4 * g + 1], t[4 * g + 2], t[4 * g + 3]};
                        *(f32x4*)(stg + ml * SROW + (8 * g + 4 * nh) * 4) = v;
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                    for (int pass = 0; pass < 4; ++pass) {
                        const int row = pass * 8 + (lane >> 3), piece = lane & 7;
                        f32x4 v = *(const f32x4*)(stg + row * SROW + piece * 16);
                        const int gm = m0 + wm * 128 + i * 32 + row;
                        const int gn = wave_n0 + j * 32 + piece * 4;
                        if (!HALF && p.partial != nullptr) {
                            // K is split: this workgroup's sums go to its plane of the workspace as they are
                            if (gm < M && gn < N) {
                                float* pp = p.partial + ((int64_t)(logical % splits) * M + gm) * N + gn;
                                if ((N & 3) == 0 && gn + 4 <= N) *(f32x4*)pp = v;
                                else
                                    for (int c = 0; c < 4; ++c)
                                        if (gn + c < N) pp[c] = v[c];
                            }
                        } else if (gm < M && gn < N) {
                            float* hp = p.h + (int64_t)gm * N + gn;
                            if (aligned && gn + 4 <= N) {
                                f32x4 hv = p.overwrite ? f32x4{0.f, 0.f, 0.f, 0.f} : ahead ? hq[DEEP ? i & 1 : 0][j][pass] : *(const f32x4*)hp;
#pragma unroll
                                for (int c = 0; c < 4; ++c) {
                                    hv[c] += v[c] + (p.bias != nullptr ? p.bias[gn + c] : 0.f);
                                    sq[pass] += hv[c] * hv[c];
                                }
                                *(f32x4*)hp = hv;
                                if (p.weighted != nullptr) {
                                    bf16x4 wv;
#pragma unroll
                                    for (int c = 0; c < 4; ++c) wv[c] = (bf16)(p.norm_w[gn + c] * hv[c]);
                                    *(bf16x4*)(p.weighted + (int64_t)gm * N + gn) = wv;
                                }
                            } else {
                                for (int c = 0; c < 4; ++c)
                                    if (gn + c < N) {
                                        const float hv = (p.overwrite ? 0.f : hp[c]) + v[c] + (p.bias != nullptr ? p.bias[gn + c] : 0.f);
                                        hp[c] = hv;
                                        sq[pass] += hv * hv;
                                        if (p.weighted != nullptr) p.weighted[(int64_t)gm * N + gn + c] = (bf16)(p.norm_w[gn + c] * hv);
                                    }
                            }
                        }
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                }
                if (p.stats_out != nullptr && (HALF || p.partial == nullptr)) {
                    // the 8 lanes of a row add their squares in a fixed order
#pragma unroll
                    for (int pass = 0; pass < 4; ++pass) {
                        float v = sq[pass];
#pragma unroll
                        for (int off = 4; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
                        const int gm = m0 + wm * 128 + i * 32 + pass * 8 + (lane >> 3);
                        if ((lane & 7) == 0 && gm < M) p.stats_out[(int64_t)stats_row * p.stats_width + gm] = v;
                    }
                }
            }
        }

        if (!has_next) break;
        // the staging is read
        __syncthreads();
        if constexpr (HALF) {
            // slots 3 and 4 take the next tile's B1 and A2
#pragma unroll
            for (int q = 3; q < 5; ++q)
#pragma unroll
                for (int i = 0; i < LA; ++i) issue_piece(q, q, i);
        } else {
            // (streamed) the next segment from its first stages on
            aim(next_unit);
#pragma unroll
            for (int st = 0; st < S - 1; ++st)
#pragma unroll
                for (int i = 0; i < L; ++i) issue_stage(st, st, i);
        }
        logical = next;
        unit = next_unit;
    }
}

// The end of the residual form where K was split: h += sum over the splits (in split order) + bias, the next norm's
// weighted rows and the sums of squares, laid out as the unsplit kernel's (one row of the statistics per 64
// columns).  A workgroup takes 16 rows x 64 columns (blockIdx.x counts the rows of the statistics); the 16 lanes of
// a row read 256 consecutive bytes of a plane.
__global__ void __launch_bounds__(256)
big_split_reduce_kernel(const BigArgs p) {
    const int row = threadIdx.x >> 4, cg = threadIdx.x & 15;
    const int gm = blockIdx.y * 16 + row, gn = blockIdx.x * 64 + cg * 4;
    const int M = p.M, N = p.N;
    const bool whole = (N & 3) == 0 && ((uintptr_t)p.h & 15) == 0 && (p.weighted == nullptr || ((uintptr_t)p.weighted & 7) == 0);
    float sq = 0.f;
    if (gm < M && gn < N) {
        const bool four = whole && gn + 4 <= N;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        const float* pp = p.partial + (int64_t)gm * N + gn;
        const int64_t plane = (int64_t)M * N;
        if (four) {
            // four planes' loads in flight at a time, added in split order
            int s = 0;
            for (; s + 4 <= p.splits; s += 4) {
                const f32x4 a = *(const f32x4*)(pp + s * plane), b = *(const f32x4*)(pp + (s + 1) * plane);
                const f32x4 c = *(const f32x4*)(pp + (s + 2) * plane), d = *(const f32x4*)(pp + (s + 3) * plane);
                sum += a;
                sum += b;
                sum += c;
                sum += d;
            }
            for (; s < p.splits; ++s) sum += *(const f32x4*)(pp + s * plane);
        } else {
            for (int s = 0; s < p.splits; ++s)
                for (int c = 0; c < 4; ++c)
                    if (gn + c < N) sum[c] += pp[s * plane + c];
        }
        float* hp = p.h + (int64_t)gm * N + gn;
        if (four) {
            f32x4 hv = p.overwrite ? f32x4{0.f, 0.f, 0.f, 0.f} : *(const f32x4*)hp;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                hv[c] += sum[c] + (p.bias != nullptr ? p.bias[gn + c] : 0.f);
                sq += hv[c] * hv[c];
            }
            *(f32x4*)hp = hv;
            if (p.weighted != nullptr) {
                bf16x4 wv;
#pragma unroll
                for (int c = 0; c < 4; ++c) wv[c] = (bf16)(p.norm_w[gn + c] * hv[c]);
                *(bf16x4*)(p.weighted + (int64_t)gm * N + gn) = wv;
            }
        } else {
            for (int c = 0; c < 4; ++c)
                if (gn + c < N) {
                    const float hv = (p.overwrite ? 0.f : hp[c]) + sum[c] + (p.bias != nullptr ? p.bias[gn + c] : 0.f);
                    hp[c] = hv;
                    sq += hv * hv;
                    if (p.weighted != nullptr) p.weighted[(int64_t)gm * N + gn + c] = (bf16)(p.norm_w[gn + c] * hv);
                }
        }
    }
    if (p.stats_out != nullptr) {
        // the 16 lanes of a row add their squares in a fixed order; every lane takes part.  Columns past N inside
        // the last tile give a row of zeros, as the unsplit kernel leaves it.
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
        if (cg == 0 && gm < M) p.stats_out[(int64_t)blockIdx.x * p.stats_width + gm] = sq;
    }
}

// The end of the plain form where K was split: out = s[m] * (sum over the splits, in split order) + bias -> bfloat16.
// A workgroup takes 16 rows x 64 columns, as big_split_reduce_kernel does.
__global__ void __launch_bounds__(256)
big_split_reduce_plain_kernel(const BigArgs p) {
    const int row = threadIdx.x >> 4, cg = threadIdx.x & 15;
    const int gm = blockIdx.y * 16 + row, gn = blockIdx.x * 64 + cg * 4;
    const int M = p.M, N = p.N;
    if (gm >= M || gn >= N) return;
    const bool four = (N & 3) == 0 && (p.ldo & 3) == 0 && ((uintptr_t)p.out & 7) == 0 && gn + 4 <= N;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    const float* pp = p.partial + (int64_t)gm * N + gn;
    const int64_t plane = (int64_t)M * N;
    if (four) {
        int s = 0;
        for (; s + 4 <= p.splits; s += 4) {
            const f32x4 a = *(const f32x4*)(pp + s * plane), b = *(const f32x4*)(pp + (s + 1) * plane);
            const f32x4 c = *(const f32x4*)(pp + (s + 2) * plane), d = *(const f32x4*)(pp + (s + 3) * plane);
            sum += a;
            sum += b;
            sum += c;
            sum += d;
        }
        for (; s < p.splits; ++s) sum += *(const f32x4*)(pp + s * plane);
    } else {
        for (int s = 0; s < p.splits; ++s)
            for (int c = 0; c < 4; ++c)
                if (gn + c < N) sum[c] += pp[s * plane + c];
    }
    const float scale = p.row_scale != nullptr ? p.row_scale[gm] : 1.f;
    bf16* op = p.out + (int64_t)gm * p.ldo + gn;
    if (four) {
        bf16x4 v;
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = (bf16)big_scale_bias(scale, sum[c], p.bias != nullptr ? p.bias[gn + c] : 0.f);
        *(bf16x4*)op = v;
    } else {
        for (int c = 0; c < 4; ++c)
            if (gn + c < N) op[c] = (bf16)big_scale_bias(scale, sum[c], p.bias != nullptr ? p.bias[gn + c] : 0.f);
    }
}

// The end of a streamed product for the tiles whose K more than one workgroup walked.  The boundary between the
// ranges of workgroup b - 1 and workgroup b (blockIdx.x = b - 1) that lies inside a tile, and is the first to do so,
// stands for that tile: a workgroup takes 16 of the tile's rows (blockIdx.y), adds the tile's segments in stage
// order (the slots of the workgroups b - 1, b, ... while their ranges begin inside the tile) and ends as the form's
// epilogue does: plain (row scale, bias, bfloat16), gated, or into the stream / float32 with the next norm's rows and
// the sums of squares (one row of the statistics per 64 columns, as the epilogue lays them out).
template <int BM, int BN>
__global__ void __launch_bounds__(256)
big_stream_finish_kernel(const BigArgs p, int epi) {
    const int W = p.stream_wgs, M = p.M, N = p.N;
    const int KTF = (p.K + BIG_BK - 1) / BIG_BK;
    const int64_t units = (int64_t)p.tiles_m * p.tiles_n * KTF;
    const int b = blockIdx.x + 1;
    const int64_t at = units * b / W;
    if (at % KTF == 0) return;                                    // the ranges meet between two tiles
    const int tile = (int)(at / KTF);
    const int64_t tile_first = (int64_t)tile * KTF, tile_end = tile_first + KTF;
    if (units * (b - 1) / W > tile_first) return;                 // an earlier boundary stands for this tile
    const int tn = tile / p.tiles_m, tm = tile % p.tiles_m;
    const int row = threadIdx.x >> 4, cg = threadIdx.x & 15;
    const int rt = blockIdx.y * 16 + row, gm = tm * BM + rt;
    constexpr int QUADS = BN / 64;                                // quads of columns a thread takes: 64 columns apart
    f32x4 sum[QUADS];
#pragma unroll
    for (int q = 0; q < QUADS; ++q) sum[q] = f32x4{0.f, 0.f, 0.f, 0.f};
    // In the gated form a thread needs the gate and the up value of a channel: quad q of thread cg is then the
    // quad (q * 16 + cg) of the row's BN / 8 (gate quad, up quad) pairs instead of the columns 64 q + 4 cg.
    auto column = [&](int q) { return epi == BIG_SWIGLU ? ((q * 16 + cg) >> 2) * 32 + ((q * 16 + cg) & 3) * 4 : q * 64 + cg * 4; };
    f32x4 up[QUADS];
#pragma unroll
    for (int q = 0; q < QUADS; ++q) up[q] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int w = b - 1; w < W; ++w) {
        const int64_t first = units * w / W, end = units * (w + 1) / W;
        if (first >= tile_end) break;
        if (first >= end) continue;                               // a workgroup without units left nothing
        const float* slot = p.slots + ((int64_t)w * 2 + (first < tile_first ? 1 : 0)) * (BM * BN) + rt * BN;
#pragma unroll
        for (int q = 0; q < QUADS; ++q) {
            if (epi == BIG_SWIGLU && q >= QUADS / 2) break;
            const int c = column(q);
            sum[q] += *(const f32x4*)(slot + c);
            if (epi == BIG_SWIGLU) up[q] += *(const f32x4*)(slot + c + 16);
        }
    }
    if (epi == BIG_PLAIN || epi == BIG_SWIGLU) {
        if (gm >= M) return;
        const float scale = p.row_scale != nullptr ? p.row_scale[gm] : 1.f;
        const int out_n = epi == BIG_SWIGLU ? N / 2 : N;
        const bool aligned = (out_n & 3) == 0 && (p.ldo & 3) == 0 && ((uintptr_t)p.out & 7) == 0;
#pragma unroll
        for (int q = 0; q < QUADS; ++q) {
            if (epi == BIG_SWIGLU && q >= QUADS / 2) break;
            const int c = column(q);
            const int gn = tn * BN + c;                           // first of the four columns of the product
            if (gn >= N) continue;
            bf16x4 v;
            int gc;                                               // first output column
            if (epi == BIG_SWIGLU) {
                gc = (tn * BN + (c >> 5) * 32) / 2 + (c & 15);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float gate = scale * sum[q][e], u = scale * up[q][e];
                    v[e] = (bf16)big_silu_mul(gate, u);
                }
            } else {
                gc = gn;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (bf16)big_scale_bias(scale, sum[q][e], p.bias != nullptr && gn + e < N ? p.bias[gn + e] : 0.f);
            }
            bf16* dst = p.out + (int64_t)gm * p.ldo + gc;
            if (aligned && gc + 4 <= out_n) *(bf16x4*)dst = v;
            else
                for (int e = 0; e < 4; ++e)
                    if (gc + e < out_n) dst[e] = v[e];
        }
        return;
    }
    // into the stream (or float32 results as they are)
    const bool aligned = (N & 3) == 0 && ((uintptr_t)p.h & 15) == 0 && (p.weighted == nullptr || ((uintptr_t)p.weighted & 7) == 0);
#pragma unroll
    for (int q = 0; q < QUADS; ++q) {
        const int gn = tn * BN + q * 64 + cg * 4;
        float sq = 0.f;
        if (gm < M && gn < N) {
            float* hp = p.h + (int64_t)gm * N + gn;
            if (aligned && gn + 4 <= N) {
                f32x4 hv = p.overwrite ? f32x4{0.f, 0.f, 0.f, 0.f} : *(const f32x4*)hp;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    hv[e] += sum[q][e] + (p.bias != nullptr ? p.bias[gn + e] : 0.f);
                    sq += hv[e] * hv[e];
                }
                *(f32x4*)hp = hv;
                if (p.weighted != nullptr) {
                    bf16x4 wv;
#pragma unroll
                    for (int e = 0; e < 4; ++e) wv[e] = (bf16)(p.norm_w[gn + e] * hv[e]);
                    *(bf16x4*)(p.weighted + (int64_t)gm * N + gn) = wv;
                }
            } else {
                for (int e = 0; e < 4; ++e)
                    if (gn + e < N) {
                        const float hv = (p.overwrite ? 0.f : hp[e]) + sum[q][e] + (p.bias != nullptr ? p.bias[gn + e] : 0.f);
                        hp[e] = hv;
                        sq += hv * hv;
                        if (p.weighted != nullptr) p.weighted[(int64_t)gm * N + gn + e] = (bf16)(p.norm_w[gn + e] * hv);
                    }
            }
        }
        if (p.stats_out != nullptr) {
            // the 16 lanes of a row add their squares in a fixed order; every lane takes part
#pragma unroll
            for (int off = 8; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
            if (cg == 0 && gm < M) p.stats_out[(int64_t)(tn * QUADS + q) * p.stats_width + gm] = sq;
        }
    }
}

// The end of the gated form where K was split: out = silu(s g) * (s u) with g and u the sums over the splits (in split
// order) of a channel's gate and up columns, which lie 16 apart in blocks of 32 columns.  A workgroup takes 16 rows x
// 128 columns of the product (64 of the output); a lane adds four gate columns and their four up columns.
__global__ void __launch_bounds__(256)
big_split_reduce_swiglu_kernel(const BigArgs p) {
    const int row = threadIdx.x >> 4, cg = threadIdx.x & 15;
    const int gm = blockIdx.y * 16 + row;
    const int gn = blockIdx.x * 128 + (cg >> 2) * 32 + (cg & 3) * 4;      // first of the four gate columns
    const int M = p.M, N = p.N;
    if (gm >= M || gn >= N) return;
    f32x4 gate = {0.f, 0.f, 0.f, 0.f}, up = gate;
    const float* pp = p.partial + (int64_t)gm * N + gn;
    const int64_t plane = (int64_t)M * N;
    for (int sp = 0; sp < p.splits; ++sp) {
        gate += *(const f32x4*)(pp + sp * plane);
        up += *(const f32x4*)(pp + sp * plane + 16);
    }
    const float scale = p.row_scale != nullptr ? p.row_scale[gm] : 1.f;
    bf16x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (bf16)big_silu_mul(scale * gate[e], scale * up[e]);
    const int gc = (gn >> 5) * 16 + (gn & 15);
    bf16* dst = p.out + (int64_t)gm * p.ldo + gc;
    if ((p.ldo & 3) == 0 && ((uintptr_t)p.out & 7) == 0) *(bf16x4*)dst = v;
    else
        for (int e = 0; e < 4; ++e) dst[e] = v[e];
}

// The end of the q/k/v product where K was split: the splits' sums, added in split order, scaled per row, plus the
// bias, rounded to bfloat16, then what the rotary encoding and the cache store do in a kernel of their own elsewhere
// (rope_kv.hip, and the end of the few-rows q/k/v product in linear_fused.hip, whose rounding this follows: the sum is
// rounded before it is rotated, so k in the cache does not depend on which kernel wrote it): q and k heads are rotated
// by the token's position (x' = x cos + rotate_half(x) sin, channels j and j + D/2 together), q goes to out
// [M, nq D], k and v to their pages (v transposed inside a page).  A workgroup takes one head of 16 rows; a thread
// the channels j .. j + 3 and j + D/2 .. of a row.
// Reference: somi_inference/models/qwen2.py:95-113, 286-293; core/paged_attention.py:246-292.
__global__ void __launch_bounds__(256)
big_split_reduce_rope_kernel(const BigArgs p) {
    const int row = threadIdx.x >> 4, lane = threadIdx.x & 15;
    const int gm = blockIdx.y * 16 + row, head = blockIdx.x;
    const int M = p.M, N = p.N, D = p.D, half = D / 2, nq = p.nq, nkv = p.nkv;
    if (gm >= M) return;
    const float scale = p.row_scale != nullptr ? p.row_scale[gm] : 1.f;
    const int64_t plane = (int64_t)M * N;
    const float pos = (float)p.positions[gm];
    const int slot = p.cache_slots[gm];
    for (int j = lane * 4; j < half; j += 64) {
        const int gn = head * D + j;
        const float* pp = p.partial + (int64_t)gm * N + gn;
        f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = lo;
        for (int sp = 0; sp < p.splits; ++sp) {
            lo += *(const f32x4*)(pp + sp * plane);
            hi += *(const f32x4*)(pp + sp * plane + half);
        }
        bf16x4 first, second;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float x1 = (float)(bf16)big_scale_bias(scale, lo[e], p.bias != nullptr ? p.bias[gn + e] : 0.f);
            const float x2 = (float)(bf16)big_scale_bias(scale, hi[e], p.bias != nullptr ? p.bias[gn + half + e] : 0.f);
            if (head < nq + nkv) {
                const float angle = pos * p.inv_freq[j + e];
                const float c = cosf(angle), sn = sinf(angle);
                first[e] = (bf16)(x1 * c - x2 * sn);
                second[e] = (bf16)(x2 * c + x1 * sn);
            } else {
                first[e] = (bf16)x1;
                second[e] = (bf16)x2;
            }
        }
        if (head < nq) {
            bf16* to = p.out + (int64_t)gm * nq * D + head * D + j;
            *(bf16x4*)to = first;
            *(bf16x4*)(to + half) = second;
            continue;
        }
        if (slot < 0) continue;
        const int64_t page = slot / p.page_size, off = slot % p.page_size;
        if (head < nq + nkv) {
            bf16* to = p.k_cache + ((page * nkv + (head - nq)) * p.page_size + off) * D + j;
            *(bf16x4*)to = first;
            *(bf16x4*)(to + half) = second;
        } else {
            bf16* to = p.v_cache + ((page * nkv + (head - nq - nkv)) * D + j) * p.page_size + off;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                to[(int64_t)e * p.page_size] = first[e];
                to[(int64_t)(half + e) * p.page_size] = second[e];
            }
        }
    }
}

// ---------------------------------------------------------------------- host side
static int big_compute_units() { return somi_units(); }

// Streaming (BigArgs.stream_wgs) is there for the asking (tile code + BIG_TILE_STREAM) and is never chosen: measured at
// 7B layer sizes on an MI355X it loses to whole tiles, or to tiles that share their K in turns, at every number of
// rows.  With equal contiguous ranges of units the workgroups of a die no longer walk the row tiles of a column tile
// in step, so a weight tile is no longer read from memory once and from the L2 seven times (2,048 rows: q/k/v 110 us
// against 83, down 343 against 243, gate_up 629 against 494, the slots' traffic included); with one row tile, where
// nothing is shared, a stage of a workgroup takes as long as its loads' latency, and twice the workgroups wait
// twice as long (gate_up at 256 rows: 110 us against 104).
#define BIG_STREAM_MIN_STAGES 1          // stages a workgroup gets at least where streaming is asked for
static bool big_streams(int tiles, int k, int cus) {
    (void)tiles; (void)k; (void)cus;
    return false;
}

// The wide tile moves fewer bytes per product and wins where it fills the device; the narrow one has twice the
// workgroups.  Costs in units of a narrow tile's time: rounds of tiles x the tile's size (the narrow tile is
// about 8 % less efficient per product).
static bool big_use_wide(int m, int n, int k, int cus = 0) {
    (void)k;
    if (cus <= 0) cus = big_compute_units();
    const int tm = ceil_div(m, BIG_BM);
    const double wide = (double)ceil_div(tm * ceil_div(n, 256), cus) * 2.0;
    const double narrow = (double)ceil_div(tm * ceil_div(n, 128), cus) * 1.08;
    return wide <= narrow;
}

// The 128-row tile: asked for (tile code BIG_TILE_LOW), or chosen for up to 128 rows.
#define BIG_TILE_LOW 1
static bool big_use_low(int m, int tile) { return tile == BIG_TILE_LOW || (tile == 0 && m <= 128); }
// A tile code may carry a word on streaming: + BIG_TILE_STREAM asks for it, + BIG_TILE_NO_STREAM forbids it
// (measurements and tests of each tile shape either way); without, the launcher chooses.
#define BIG_TILE_STREAM 1000
#define BIG_TILE_NO_STREAM 2000
static int big_tile_shape(int tile) { return tile % BIG_TILE_STREAM; }
static bool big_tile_code_ok(int tile) {
    const int shape = big_tile_shape(tile);
    return tile >= 0 && tile < 3 * BIG_TILE_STREAM && (shape == 0 || shape == BIG_TILE_LOW || shape == 128 || shape == 256);
}

template <int BM, int BN, int S, int NW, int EPI, bool KTAIL, bool WONCE>
static int big_launch_once(const BigArgs& args, hipStream_t stream) {
    const int lds_bytes = S == 5 ? 5 * 256 * BIG_ROW_BYTES : S * (BM + BN) * BIG_ROW_BYTES;
    static bool raised[64];
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess || device < 0 || device >= 64) return somi_fail("linear_big: hipGetDevice failed");
    if (!raised[device]) {
        err = hipFuncSetAttribute((const void*)linear_big_kernel<BM, BN, S, NW, EPI, KTAIL, WONCE>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (err != hipSuccess) return somi_fail("linear_big: %d bytes of LDS refused: %s", lds_bytes, hipGetErrorString(err));
        raised[device] = true;
    }
    // one workgroup per tile; the wide form is persistent: at most one workgroup per compute unit, a multiple of 8
    // (the dies), each walking its die's tiles
    const int per = ceil_div(args.tiles_m * args.tiles_n * args.splits, 8);
    int per_die = per;
    if (S == 5) {
        const int cus_per_die = big_compute_units() / 8 > 0 ? big_compute_units() / 8 : 1;
        per_die = per < cus_per_die ? per : cus_per_die;
    }
    const int grid = args.stream_wgs > 0 ? args.stream_wgs : per_die * 8;
    hipLaunchKernelGGL((linear_big_kernel<BM, BN, S, NW, EPI, KTAIL, WONCE>), dim3(grid), dim3(NW * 64), lds_bytes, stream, args);
    SOMI_LAUNCH_CHECK("linear_big");
    if (args.stream_wgs > 1) {
        hipLaunchKernelGGL((big_stream_finish_kernel<BM, BN>), dim3(args.stream_wgs - 1, BM / 16), dim3(256), 0, stream, args, EPI);
        SOMI_LAUNCH_CHECK("linear_big: finish");
    }
    if (EPI == BIG_RESIDUAL && args.partial != nullptr) {
        if (args.reduce_plain == 2)
            hipLaunchKernelGGL(big_split_reduce_rope_kernel, dim3(args.nq + 2 * args.nkv, ceil_div(args.M, 16)), dim3(256), 0, stream, args);
        else if (args.reduce_plain == 3)
            hipLaunchKernelGGL(big_split_reduce_swiglu_kernel, dim3(ceil_div(args.N, 128), ceil_div(args.M, 16)), dim3(256), 0, stream, args);
        else if (args.reduce_plain)
            hipLaunchKernelGGL(big_split_reduce_plain_kernel, dim3(ceil_div(args.N, 64), ceil_div(args.M, 16)), dim3(256), 0, stream, args);
        else
            hipLaunchKernelGGL(big_split_reduce_kernel, dim3(args.stats_rows, ceil_div(args.M, 16)), dim3(256), 0, stream, args);
        SOMI_LAUNCH_CHECK("linear_big: reduce");
    }
    return 0;
}

// A weight that one row tile reads is read once: the 128-row tile's loads of it carry the hint (decode steps of 96
// and 128 requests 4 and 2 % shorter).  The 256-row tiles are left without: where they have one row tile it changes
// nothing inside decode steps (256 requests: 17.5 ms either way), and a weight that is still in the memory-side
// cache from the call before is read slower with it (7B q/k/v at 256 rows in a loop: 85 us against 74).
template <int BM, int BN, int S, int NW, int EPI, bool KTAIL>
static int big_launch_one(const BigArgs& args, hipStream_t stream) {
    if constexpr (BM == 128) return big_launch_once<BM, BN, S, NW, EPI, KTAIL, true>(args, stream);
    else return big_launch_once<BM, BN, S, NW, EPI, KTAIL, false>(args, stream);
}

// How many workgroups share a tile's K in the residual form (tiles of three whole stages): as many as give about
// every compute unit a workgroup, with at least BIG_SPLIT_MIN_STAGES stages each, within the workspace; 1 where the
// tiles alone fill half of the device.  (7B down projection at 192 rows: 28 tiles of 256 x 128, 296 stages: 227 us
// unsplit, 62 in 9 splits.  At least 4 stages, not 8: a K of 896 has 14, and with 8 the products of a 0.5B layer at
// 65 to 128 rows ran on the 4 or 5 workgroups of their tiles: steps of 96 / 128 requests 3.09 -> 2.63 / 3.30 -> 2.74
// ms; at 7B sizes nothing changes.)
#define BIG_SPLIT_MIN_STAGES 4
static int big_splits(int tiles, int m, int n, int k, int64_t workspace_floats, int cus = 0) {
    if (cus <= 0) cus = big_compute_units();
    const int stages = ceil_div(k, BIG_BK);
    if (workspace_floats <= 0 || tiles * 2 > cus) return 1;
    int64_t splits = cus / tiles;
    if (splits > stages / BIG_SPLIT_MIN_STAGES) splits = stages / BIG_SPLIT_MIN_STAGES;
    if (splits > workspace_floats / ((int64_t)m * n)) splits = workspace_floats / ((int64_t)m * n);
    if (splits <= 1) return 1;
    const int per = ceil_div(stages, (int)splits);
    return ceil_div(stages, per);                    // no split without stages
}

template <int EPI>
static int big_launch(BigArgs& args, int tile, hipStream_t stream, float* workspace = nullptr, int64_t workspace_floats = 0) {
    const bool ktail = args.K % BIG_BK != 0;
    const int shape = big_tile_shape(tile), word = tile - shape;
    const int cus = big_compute_units();
    args.splits = 1;
    args.partial = nullptr;
    args.stream_wgs = 0;
    args.slots = nullptr;
    auto split_k = [&]() {                     // the tiles are set: share their K where they are few
        if (EPI != BIG_RESIDUAL || workspace == nullptr || word == BIG_TILE_STREAM) return;
        args.splits = big_splits(args.tiles_m * args.tiles_n, args.M, args.N, args.K, workspace_floats);
        if (args.splits > 1) args.partial = workspace;
    };
    auto stream_units = [&](int bm, int bn) {  // or deal out (tile, stage) units where the tiles' rounds leave units idle
        if (workspace == nullptr || args.splits > 1 || word == BIG_TILE_NO_STREAM) return;
        const int tiles = args.tiles_m * args.tiles_n, wgs = cus / 8 * 8;
        if (wgs < 8 || (int64_t)wgs * 2 * bm * bn > workspace_floats) return;
        if (word == BIG_TILE_STREAM ? (int64_t)tiles * ceil_div(args.K, BIG_BK) >= wgs : big_streams(tiles, args.K, cus)) {
            args.stream_wgs = wgs;
            args.slots = workspace;
        }
    };
    if (big_use_low(args.M, shape)) {
        // up to 128 rows: one row tile of 128, four wavefronts side by side over 256 columns
        args.tiles_m = ceil_div(args.M, 128);
        args.tiles_n = ceil_div(args.N, 256);
        args.stats_rows = args.tiles_n * 4;
        split_k();
        stream_units(128, 256);
        return ktail ? big_launch_one<128, 256, 3, 4, EPI, true>(args, stream) : big_launch_one<128, 256, 3, 4, EPI, false>(args, stream);
    }
    const bool wide = shape == 0 ? big_use_wide(args.M, args.N, args.K) : shape == 256;
    args.tiles_m = ceil_div(args.M, BIG_BM);
    args.tiles_n = ceil_div(args.N, wide ? 256 : 128);
    args.stats_rows = wide ? args.tiles_n * 4 : args.tiles_n * 2;
    if (!wide) split_k();
    if (wide || word == BIG_TILE_STREAM) stream_units(BIG_BM, wide ? 256 : 128);
    if (wide) return ktail ? big_launch_one<256, 256, 5, 8, EPI, true>(args, stream) : big_launch_one<256, 256, 5, 8, EPI, false>(args, stream);
    return ktail ? big_launch_one<256, 128, 3, 4, EPI, true>(args, stream) : big_launch_one<256, 128, 3, 4, EPI, false>(args, stream);
}

static int big_check(const char* what, const void* x, int64_t ldx, const void* w, int64_t ldw, int m, int n, int k) {
    SOMI_REQUIRE(m > 0 && n > 0 && k > 0, "%s: bad sizes m=%d n=%d k=%d", what, m, n, k);
    SOMI_REQUIRE(k % 8 == 0, "%s: K = %d is no multiple of 8", what, k);
    SOMI_REQUIRE(ldx >= k && ldw >= k && ldx % 8 == 0 && ldw % 8 == 0, "%s: row strides %lld and %lld must be multiples of 8 and >= K",
                 what, (long long)ldx, (long long)ldw);
    SOMI_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0, "%s: operands must be aligned to 16 bytes", what);
    // a lane's byte offset inside a tile is 32-bit
    SOMI_REQUIRE((int64_t)256 * ldx * 2 < ((int64_t)1 << 32) && (int64_t)256 * ldw * 2 < ((int64_t)1 << 32),
                 "%s: rows too long for 32-bit offsets inside a tile", what);
    return 0;
}

// s[m] = 1 / sqrt(sum_b stats[b][m] / k + eps): the scale an RMS norm gives row m, from the partial sums of squares
// that the residual forms leave (here and in linear_fused.hip).  A workgroup takes 8 rows; thread (row, e) adds the
// blocks b = e, e + 32, e + 64, ... in that order, and the 32 sums of a row are added as a fixed tree, so a row's
// scale does not depend on how many rows there are.  (Some hundred blocks of a few-rows producer, 128 rows: 8 us with
// 32 rows a workgroup, where four workgroups walked 28 blocks a thread.)
#define ROW_SCALE_ROWS 8
__global__ void __launch_bounds__(256)
row_scale_kernel(const float* __restrict__ stats, int blocks, int width, int m, float inv_k, float eps, float* __restrict__ out) {
    __shared__ float parts[32][ROW_SCALE_ROWS + 1];
    const int r = threadIdx.x & (ROW_SCALE_ROWS - 1), e = threadIdx.x / ROW_SCALE_ROWS;
    const int row = blockIdx.x * ROW_SCALE_ROWS + r;
    float part = 0.f;
    if (row < m)
        for (int b = e; b < blocks; b += 32) part += stats[(int64_t)b * width + row];
    parts[e][r] = part;
    __syncthreads();
    // pairs 16 apart, then 8, 4, 2, 1: the same tree for every row
    for (int half = 16; half > 0; half >>= 1) {
        if (e < half) parts[e][r] += parts[e + half][r];
        __syncthreads();
    }
    if (e == 0 && row < m) out[row] = rsqrtf(parts[0][r] * inv_k + eps);
}

extern "C" int somi_row_scale(const float* stats, int blocks, int width, int m, int k, float eps, float* out, hipStream_t stream) {
    SOMI_REQUIRE(stats != nullptr && out != nullptr && blocks > 0 && m > 0 && width >= m && k > 0,
                 "row_scale: bad arguments (blocks=%d width=%d m=%d k=%d)", blocks, width, m, k);
    hipLaunchKernelGGL(row_scale_kernel, dim3(ceil_div(m, ROW_SCALE_ROWS)), dim3(256), 0, stream, stats, blocks, width, m, 1.f / (float)k, eps, out);
    SOMI_LAUNCH_CHECK("row_scale");
    return 0;
}

// Workgroup columns that write row statistics in the residual form: the first size of stats_out.
// tile: 0 lets the launcher choose (the 128-row tile up to 128 rows, else 256-row tiles of the width that fills the
// device better); 128 or 256 asks for that width of the 256-row tile, 1 for the 128-row tile (128 x 256).
extern "C" int somi_linear_big_stats_blocks(int m, int n, int k, int tile) {
    tile = big_tile_shape(tile);
    if (big_use_low(m, tile)) return ceil_div(n, 256) * 4;
    const bool wide = tile == 0 ? big_use_wide(m, n, k) : tile == 256;
    return wide ? ceil_div(n, 256) * 4 : ceil_div(n, 128) * 2;
}

// Workgroups that share a tile's K in somi_linear_big_residual with this much workspace (1: K is not split).
extern "C" int somi_linear_big_splits(int m, int n, int k, int tile, int64_t workspace_floats) {
    if (tile - big_tile_shape(tile) == BIG_TILE_STREAM) return 1;
    tile = big_tile_shape(tile);
    if (big_use_low(m, tile)) return big_splits(ceil_div(m, 128) * ceil_div(n, 256), m, n, k, workspace_floats);
    const bool wide = tile == 0 ? big_use_wide(m, n, k) : tile == 256;
    return wide ? 1 : big_splits(ceil_div(m, BIG_BM) * ceil_div(n, 128), m, n, k, workspace_floats);
}

// Workgroups that the product's (tile, stage) units are dealt out to with this much workspace, as the entry points
// choose (0: the tiles are handed out whole), for a device of `units` compute units (0: the current device).
extern "C" int somi_linear_big_streams(int m, int n, int k, int tile, int64_t workspace_floats, int units) {
    const int cus = units > 0 ? units : big_compute_units();
    const int shape = big_tile_shape(tile), word = tile - shape;
    if (word == BIG_TILE_NO_STREAM) return 0;
    int bm = 256, bn = 128, tiles;
    bool may = false;
    if (big_use_low(m, shape)) {
        bm = 128; bn = 256; tiles = ceil_div(m, 128) * ceil_div(n, 256);
        may = big_splits(tiles, m, n, k, workspace_floats) <= 1 || word == BIG_TILE_STREAM;
    } else {
        const bool wide = shape == 0 ? big_use_wide(m, n, k, cus) : shape == 256;
        bn = wide ? 256 : 128;
        tiles = ceil_div(m, BIG_BM) * ceil_div(n, bn);
        may = wide || word == BIG_TILE_STREAM;
    }
    const int wgs = cus / 8 * 8;
    if (!may || wgs < 8 || (int64_t)wgs * 2 * bm * bn > workspace_floats) return 0;
    const bool yes = word == BIG_TILE_STREAM ? (int64_t)tiles * ceil_div(k, BIG_BK) >= wgs : big_streams(tiles, k, cus);
    return yes ? wgs : 0;
}

// The tail of a product whose 256 x 128 tiles do not come out even over the compute units: the whole rounds of tiles run
// as they are, and the column tiles that are left, too few to fill the device, share their K among workgroups as a
// product of their own over the last columns (float32 sums in the workspace, ended by a reduce kernel).  7B gate_up at
// 512 rows: two rounds and 80 tiles in 3 splits instead of three rounds, 142 us against 151 (and 160 for two rounds of
// 256 x 256 tiles).  Only from two whole rounds on: after one round the tail's two launches cost what they save, and
// one round of 256 x 256 tiles is faster than either (q/k/v at 2,048 rows: 88 us with a tail, 89 in two rounds, 78 on
// 144 tiles of 256 x 256; gate_up at 256 rows: 87, 97, 76).
// Returns the columns of the tail (0: the product runs whole) and its splits.  Costs in rounds of 256 x 128 tiles:
// a round of 256 x 256 tiles counts 1.72 (91 us against 53 over K = 3,584), the tail's launches 0.45.
static int big_tail(int m, int n, int k, int64_t workspace_floats, int cus, int* splits_out) {
    if (cus <= 0) cus = big_compute_units();
    *splits_out = 1;
    if (m <= 128 || workspace_floats <= 0) return 0;
    const int tiles_m = ceil_div(m, BIG_BM), col_tiles = ceil_div(n, 128), tiles = tiles_m * col_tiles;
    if (tiles <= cus) return 0;
    const int main_cols = (tiles / cus) * cus / tiles_m;            // column tiles of the whole rounds
    const int tail_cols = col_tiles - main_cols, tail_tiles = tail_cols * tiles_m;
    if (tail_tiles == 0 || main_cols == 0) return 0;
    const int tail_n = n - main_cols * 128;
    const int splits = big_splits(tail_tiles, m, tail_n, k, workspace_floats, cus);
    if (splits < 2) return 0;
    if (tiles / cus < 2) return 0;
    const double whole_wide = (double)ceil_div(tiles_m * ceil_div(n, 256), cus) * 1.72;
    const double whole_narrow = (double)ceil_div(tiles, cus);
    const double with_tail = (double)(main_cols * tiles_m) / cus + 1.0 / splits + 0.45;
    if (with_tail >= 0.97 * (whole_wide < whole_narrow ? whole_wide : whole_narrow)) return 0;
    *splits_out = splits;
    return tail_n;
}

// What somi_linear_big does with the last columns of a product at tile code 0 on a device of `units` compute units
// (0: the current device): the columns that run as a product of their own with K shared (0: none), and in how many
// splits.
extern "C" int somi_linear_big_tail(int m, int n, int k, int64_t workspace_floats, int units, int* splits) {
    int s = 1;
    const int tail = big_tail(m, n, k, workspace_floats, units, &s);
    if (splits != nullptr) *splits = s;
    return tail;
}

// out = s * (x . w^T) + bias -> bfloat16 [M, N]; with swiglu w is [N, K] with gate and up rows interleaved in blocks
// of 16 and out is [M, N / 2] = silu(s g) * (s u).  row_scale (or null): s [M], see somi_row_scale.  workspace (or
// null): as in somi_linear_big_residual, for the plain form (q/k/v of some hundred rows: 72 tiles at 7B sizes).
extern "C" int somi_linear_big(const void* x, int64_t ldx, const void* w, int64_t ldw, const float* bias, void* out,
                               int m, int n, int k, const float* row_scale, int swiglu, int tile, float* workspace,
                               int64_t workspace_floats, hipStream_t stream) {
    if (big_check("linear_big", x, ldx, w, ldw, m, n, k) != 0) return 1;
    SOMI_REQUIRE(out != nullptr, "linear_big: no output");
    SOMI_REQUIRE(!swiglu || (n % 32 == 0 && bias == nullptr), "linear_big: the gated form needs N a multiple of 32 and no bias");
    SOMI_REQUIRE(big_tile_code_ok(tile), "linear_big: tile code %d (0, 1, 128 or 256, + 1000 or 2000)", tile);
    BigArgs args = {};
    args.x = (const bf16*)x; args.ldx = ldx; args.w = (const bf16*)w; args.ldw = ldw; args.bias = bias;
    args.M = m; args.N = n; args.K = k; args.out = (bf16*)out; args.ldo = swiglu ? n / 2 : n;
    args.row_scale = row_scale;
    SOMI_REQUIRE(workspace == nullptr || (((uintptr_t)workspace & 15) == 0 && workspace_floats >= 0),
                 "linear_big: the workspace must be aligned to 16 bytes");
    int tail_splits = 1;
    const int tail_n = tile == 0 && workspace != nullptr ? big_tail(m, n, k, workspace_floats, 0, &tail_splits) : 0;
    if (tail_n > 0) {
        // whole rounds of 256 x 128 tiles over the first columns, then the last columns with their K shared
        const int main_n = n - tail_n;
        BigArgs head = args;
        head.N = main_n;
        const int rc = swiglu ? big_launch<BIG_SWIGLU>(head, 128 + BIG_TILE_NO_STREAM, stream)
                              : big_launch<BIG_PLAIN>(head, 128 + BIG_TILE_NO_STREAM, stream);
        if (rc != 0) return rc;
        BigArgs tail = args;
        tail.w = args.w + (int64_t)main_n * ldw;
        tail.bias = bias != nullptr ? bias + main_n : nullptr;
        tail.N = tail_n;
        tail.out = args.out + (swiglu ? main_n / 2 : main_n);
        tail.reduce_plain = swiglu ? 3 : 1;
        return big_launch<BIG_RESIDUAL>(tail, 128 + BIG_TILE_NO_STREAM, stream, workspace, workspace_floats);
    }
    if (!swiglu && workspace != nullptr && somi_linear_big_splits(m, n, k, tile, workspace_floats) > 1) {
        // the workgroups of a tile share its K and leave float32 sums; the reduce scales, adds the bias and rounds
        args.reduce_plain = 1;
        return big_launch<BIG_RESIDUAL>(args, tile, stream, workspace, workspace_floats);
    }
    return swiglu ? big_launch<BIG_SWIGLU>(args, tile, stream, workspace, workspace_floats)
                  : big_launch<BIG_PLAIN>(args, tile, stream, workspace, workspace_floats);
}

// h += x . w^T + bias, float32 in place [M, N].  norm_w / weighted (or null): weighted = bfloat16(norm_w * h);
// stats_out (or null): [somi_linear_big_stats_blocks(m, n, tile)][stats_width] sums of squares of the new h, each over
// the 64 columns of one wavefront.  workspace (or null): workspace_floats of float32, 16-byte aligned, that let the
// 128-row tile split K over workgroups where the tiles alone leave most of the device idle (somi_linear_big_splits
// says how many ways; the 256 x 128 tiles do the same); calls that share a workspace must not overlap.
extern "C" int somi_linear_big_residual(const void* x, int64_t ldx, const void* w, int64_t ldw, const float* bias, float* h,
                                        const float* norm_w, void* weighted, float* stats_out, int stats_width,
                                        int m, int n, int k, int tile, float* workspace, int64_t workspace_floats,
                                        hipStream_t stream) {
    if (big_check("linear_big_residual", x, ldx, w, ldw, m, n, k) != 0) return 1;
    SOMI_REQUIRE(h != nullptr, "linear_big_residual: no residual stream");
    SOMI_REQUIRE((weighted == nullptr) == (norm_w == nullptr), "linear_big_residual: the norm's weight and its rows come together");
    SOMI_REQUIRE(stats_out == nullptr || stats_width >= m, "linear_big_residual: row statistics of width %d do not cover %d rows", stats_width, m);
    SOMI_REQUIRE(big_tile_code_ok(tile), "linear_big_residual: tile code %d (0, 1, 128 or 256, + 1000 or 2000)", tile);
    BigArgs args = {};
    args.x = (const bf16*)x; args.ldx = ldx; args.w = (const bf16*)w; args.ldw = ldw; args.bias = bias;
    args.M = m; args.N = n; args.K = k; args.h = h; args.norm_w = norm_w; args.weighted = (bf16*)weighted;
    args.stats_out = stats_out; args.stats_width = stats_width;
    SOMI_REQUIRE(workspace == nullptr || (((uintptr_t)workspace & 15) == 0 && workspace_floats >= 0),
                 "linear_big_residual: the workspace must be aligned to 16 bytes");
    return big_launch<BIG_RESIDUAL>(args, tile, stream, workspace, workspace_floats);
}

// out = x . w^T + bias -> float32 [M, N] (logits of many rows, which must not pass through bfloat16): the residual
// form's end writing its sums instead of adding them, without the norm's by-products.
extern "C" int somi_linear_big_f32(const void* x, int64_t ldx, const void* w, int64_t ldw, const float* bias, float* out,
                                   int m, int n, int k, int tile, float* workspace, int64_t workspace_floats,
                                   hipStream_t stream) {
    if (big_check("linear_big_f32", x, ldx, w, ldw, m, n, k) != 0) return 1;
    SOMI_REQUIRE(out != nullptr, "linear_big_f32: no output");
    SOMI_REQUIRE(big_tile_code_ok(tile), "linear_big_f32: tile code %d (0, 1, 128 or 256, + 1000 or 2000)", tile);
    BigArgs args = {};
    args.x = (const bf16*)x; args.ldx = ldx; args.w = (const bf16*)w; args.ldw = ldw; args.bias = bias;
    args.M = m; args.N = n; args.K = k; args.h = out; args.overwrite = 1;
    SOMI_REQUIRE(workspace == nullptr || (((uintptr_t)workspace & 15) == 0 && workspace_floats >= 0),
                 "linear_big_f32: the workspace must be aligned to 16 bytes");
    return big_launch<BIG_RESIDUAL>(args, tile, stream, workspace, workspace_floats);
}

// The q/k/v product of many rows with the rotary encoding of q and k and the store of k and v into their cache pages
// in its end, for the sizes at which the plain form shares a tile's K among workgroups (somi_linear_big_splits > 1
// with this workspace; refused otherwise: the caller then runs somi_linear_big and the rotation as two calls).
// w: [(nq + 2 nkv) D, K], the rows of the q heads, then the k heads, then the v heads; row_scale (or null): [M];
// q: [M, nq D] bfloat16, out, rotated; positions, slots: [M] (slot = page * page_size + offset, or -1: nothing is
// stored for the row); inv_freq: [D / 2] (the whole head is rotated); k_cache [pages, nkv, page_size, D], v_cache
// [pages, nkv, D, page_size].  D a multiple of 8.
extern "C" int somi_linear_big_rope_store(const void* x, int64_t ldx, const void* w, int64_t ldw, const float* bias, void* q,
                                          int m, int k, const float* row_scale, const int* positions, const int* slots,
                                          const float* inv_freq, void* k_cache, void* v_cache, int nq, int nkv, int D,
                                          int page_size, int tile, float* workspace, int64_t workspace_floats,
                                          hipStream_t stream) {
    SOMI_REQUIRE(nq > 0 && nkv > 0 && D > 0 && D % 8 == 0, "linear_big_rope_store: head_dim (%d) must be a multiple of 8", D);
    const int64_t columns = (int64_t)(nq + 2 * nkv) * D;
    SOMI_REQUIRE(columns < ((int64_t)1 << 30), "linear_big_rope_store: too many columns");
    const int n = (int)columns;
    if (big_check("linear_big_rope_store", x, ldx, w, ldw, m, n, k) != 0) return 1;
    SOMI_REQUIRE(q && positions && slots && inv_freq && k_cache && v_cache && page_size > 0,
                 "linear_big_rope_store: q, positions, slots, inv_freq and the caches are needed");
    SOMI_REQUIRE((uintptr_t)q % 8 == 0 && (uintptr_t)k_cache % 8 == 0, "linear_big_rope_store: q and the k cache must be 8-byte aligned");
    SOMI_REQUIRE(big_tile_code_ok(tile), "linear_big_rope_store: tile code %d (0, 1, 128 or 256, + 1000 or 2000)", tile);
    SOMI_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 15) == 0, "linear_big_rope_store: a workspace aligned to 16 bytes is needed");
    SOMI_REQUIRE(somi_linear_big_splits(m, n, k, tile, workspace_floats) > 1,
                 "linear_big_rope_store: at m=%d n=%d k=%d the product does not share K among workgroups", m, n, k);
    BigArgs args = {};
    args.x = (const bf16*)x; args.ldx = ldx; args.w = (const bf16*)w; args.ldw = ldw; args.bias = bias;
    args.M = m; args.N = n; args.K = k; args.out = (bf16*)q; args.ldo = (int64_t)nq * D; args.row_scale = row_scale;
    args.positions = positions; args.cache_slots = slots; args.inv_freq = inv_freq;
    args.k_cache = (bf16*)k_cache; args.v_cache = (bf16*)v_cache;
    args.nq = nq; args.nkv = nkv; args.D = D; args.page_size = page_size;
    args.reduce_plain = 2;
    return big_launch<BIG_RESIDUAL>(args, tile, stream, workspace, workspace_floats);
}
