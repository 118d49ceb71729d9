// Token choice from float32 logits: greedy argmax, or a draw from softmax(logits / T).
//
// Reference: somi_inference/core/sampler.py:104-114 (logits /= T when T > 0), :159-176 (T == 0: argmax,
// else float32 softmax and one multinomial draw) and :80-102 (repetition penalty: a positive logit is
// divided by the penalty, a non-positive one multiplied).  The draw here is by inverse CDF from a uniform
// number that the host derives from the request's own seed and token count, so a request's tokens do not
// depend on what else is in the batch.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

// The vocabulary is cut into chunks of SAMPLE_CHUNK entries; one workgroup per (row, chunk) finds the
// chunk's maximum, its first index and (for a draw) the chunk's softmax mass relative to that maximum.  A
// second kernel, one workgroup per row, merges the chunks in index order, locates the chunk that holds the
// target mass u * total, and walks that chunk once more to pick the entry.  Chunk boundaries depend on the
// vocabulary only, so a row's token does not depend on the batch.
#define SAMPLE_NT 256
#define SAMPLE_PER_THREAD 8
#define SAMPLE_CHUNK (SAMPLE_NT * SAMPLE_PER_THREAD)

__global__ void __launch_bounds__(SAMPLE_NT)
sample_chunks_kernel(const float* __restrict__ logits, int vocab, int chunks, const float* __restrict__ temperature,
                     float* __restrict__ part /*[rows, chunks, 3]: max, first index (as int bits), mass*/) {
    __shared__ float red[16];
    __shared__ float vals[SAMPLE_NT];
    __shared__ int idxs[SAMPLE_NT];
    const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    const float* z = logits + (int64_t)row * vocab;
    const float temp = temperature[row];
    const float inv_unit = temp > 0.f ? temp : 1.f;        // greedy compares the logits themselves
    const int begin = chunk * SAMPLE_CHUNK + tid * SAMPLE_PER_THREAD;
    float v[SAMPLE_PER_THREAD];
    float best = -INFINITY;
    int best_i = vocab;
#pragma unroll
    for (int j = 0; j < SAMPLE_PER_THREAD; ++j) {
        const int i = begin + j;
        v[j] = i < vocab ? z[i] / inv_unit : -INFINITY;
        if (i < vocab && (v[j] > best || best_i == vocab)) { best = v[j]; best_i = i; }
    }
    vals[tid] = best;
    idxs[tid] = best_i;
    __syncthreads();
    for (int step = SAMPLE_NT / 2; step > 0; step >>= 1) {
        if (tid < step) {
            const float ov = vals[tid + step];
            const int oi = idxs[tid + step];
            const bool take = oi < vocab && (idxs[tid] == vocab || ov > vals[tid] || (ov == vals[tid] && oi < idxs[tid]));
            if (take) { vals[tid] = ov; idxs[tid] = oi; }
        }
        __syncthreads();
    }
    const float chunk_max = vals[0];
    float mass = 0.f;
    if (temp > 0.f) {
#pragma unroll
        for (int j = 0; j < SAMPLE_PER_THREAD; ++j)
            if (begin + j < vocab) mass += expf(v[j] - chunk_max);
        mass = block_sum<SAMPLE_NT>(mass, red);
    }
    if (tid == 0) {
        float* p = part + ((int64_t)row * chunks + chunk) * 3;
        p[0] = chunk_max;
        p[1] = __int_as_float(idxs[0]);
        p[2] = mass;
    }
}

__global__ void __launch_bounds__(SAMPLE_NT)
sample_pick_kernel(const float* __restrict__ logits, int vocab, int chunks, const float* __restrict__ temperature,
                   const float* __restrict__ uniform, const float* __restrict__ part, int* __restrict__ out) {
    __shared__ float sums[SAMPLE_NT];
    __shared__ float s_before, s_target, s_max;
    __shared__ int s_chunk, s_owner;
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* z = logits + (int64_t)row * vocab;
    const float* p = part + (int64_t)row * chunks * 3;
    const float temp = temperature[row];
    if (tid == 0) {
        float mx = -INFINITY;
        int first = vocab;
        for (int c = 0; c < chunks; ++c)                    // chunks in index order: the first maximum wins
            if (p[c * 3] > mx || first == vocab) { mx = p[c * 3]; first = __float_as_int(p[c * 3 + 1]); }
        s_max = mx;
        if (temp == 0.f) {
            out[row] = first;
        } else {
            float total = 0.f;
            for (int c = 0; c < chunks; ++c) total += p[c * 3 + 2] * expf(p[c * 3] - mx);
            const float target = uniform[row] * total;
            float run = 0.f;
            int owner = -1, last_nonzero = 0;
            for (int c = 0; c < chunks; ++c) {
                const float mass = p[c * 3 + 2] * expf(p[c * 3] - mx);
                if (mass > 0.f) last_nonzero = c;
                if (owner < 0 && target < run + mass) { owner = c; s_before = run; }
                run += mass;
            }
            if (owner < 0) {                                // rounding pushed the target past the total
                owner = last_nonzero;
                s_before = -INFINITY;                       // take the chunk's last entry with mass
            }
            s_chunk = owner;
            s_target = target;
        }
    }
    __syncthreads();
    if (temp == 0.f) return;
    const int begin = s_chunk * SAMPLE_CHUNK + tid * SAMPLE_PER_THREAD;
    float w[SAMPLE_PER_THREAD];
    float mine = 0.f;
#pragma unroll
    for (int j = 0; j < SAMPLE_PER_THREAD; ++j) {
        w[j] = begin + j < vocab ? expf(z[begin + j] / temp - s_max) : 0.f;
        mine += w[j];
    }
    sums[tid] = mine;
    __syncthreads();
    if (tid == 0) {
        const bool overshoot = s_before == -INFINITY;
        float run = overshoot ? 0.f : s_before;
        int owner = -1, last_nonzero = 0;
        for (int k = 0; k < SAMPLE_NT; ++k) {
            const float mass = sums[k];
            sums[k] = run;
            if (mass > 0.f) last_nonzero = k;
            if (!overshoot && owner < 0 && s_target < run + mass) owner = k;
            run += mass;
        }
        s_owner = owner < 0 ? last_nonzero : owner;
    }
    __syncthreads();
    if (tid == s_owner) {
        float run = sums[tid];
        int pick = -1, last = begin;
#pragma unroll
        for (int j = 0; j < SAMPLE_PER_THREAD; ++j) {
            if (w[j] > 0.f) last = begin + j;
            run += w[j];
            if (pick < 0 && s_before != -INFINITY && run > s_target) pick = begin + j;
        }
        out[row] = pick < 0 ? last : pick;
    }
}

extern "C" int somi_sample_workspace_floats(int rows, int vocab) {
    return rows * ceil_div(vocab, SAMPLE_CHUNK) * 3;
}

// logits: [rows, vocab] float32; temperature, uniform: [rows] float32 (uniform in [0, 1)); out: [rows] int32;
// workspace: somi_sample_workspace_floats(rows, vocab) floats.
extern "C" int somi_sample(const float* logits, int rows, int vocab, const float* temperature,
                           const float* uniform, int* out, float* workspace, hipStream_t stream) {
    SOMI_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
    SOMI_REQUIRE(rows <= 65535, "sample: too many rows");
    SOMI_REQUIRE(workspace != nullptr || rows == 0, "sample: a workspace is needed");
    if (rows == 0) return 0;
    const int chunks = ceil_div(vocab, SAMPLE_CHUNK);
    hipLaunchKernelGGL(sample_chunks_kernel, dim3(chunks, rows), dim3(SAMPLE_NT), 0, stream, logits, vocab, chunks,
                       temperature, workspace);
    SOMI_LAUNCH_CHECK("sample_chunks");
    hipLaunchKernelGGL(sample_pick_kernel, dim3(rows), dim3(SAMPLE_NT), 0, stream, logits, vocab, chunks, temperature,
                       uniform, workspace, out);
    SOMI_LAUNCH_CHECK("sample_pick");
    return 0;
}

// The workspace of somi_sample_no_alloc: one array per GPU, held until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; the address it yields differs from GPU to GPU and is
// what the kernels get.
static __device__ __align__(256) float scratch[SOMI_SAMPLE_SCRATCH_FLOATS];

#define SOMI_MAX_DEVICES 64
static float* g_scratch_ptr[SOMI_MAX_DEVICES];      // the array's address on each device, once asked for
static std::mutex g_scratch_mutex;

// The address of `scratch` on the current device (asked for once per device, with that device current).
static int scratch_on_current_device(float** ptr) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    SOMI_REQUIRE(err == hipSuccess, "sample_no_alloc: hipGetDevice: %s", hipGetErrorString(err));
    SOMI_REQUIRE(device >= 0 && device < SOMI_MAX_DEVICES, "sample_no_alloc: device %d is beyond the %d this library "
                 "keeps a workspace for", device, SOMI_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    if (g_scratch_ptr[device] == nullptr) {
        float* found = nullptr;
        err = hipGetSymbolAddress((void**)&found, HIP_SYMBOL(scratch));
        SOMI_REQUIRE(err == hipSuccess && found != nullptr, "sample_no_alloc: hipGetSymbolAddress on device %d: %s",
                     device, hipGetErrorString(err));
        g_scratch_ptr[device] = found;
    }
    *ptr = g_scratch_ptr[device];
    return 0;
}

extern "C" int somi_sample_no_alloc_capacity() { return SOMI_SAMPLE_SCRATCH_FLOATS; }

extern "C" int somi_sample_no_alloc(const float* logits, int rows, int vocab, const float* temperature,
                                    const float* uniform, int* out, hipStream_t stream) {
    SOMI_REQUIRE(rows >= 0 && vocab > 0, "sample_no_alloc: bad sizes rows=%d vocab=%d", rows, vocab);
    SOMI_REQUIRE(rows <= 65535, "sample_no_alloc: too many rows");
    if (rows == 0) return 0;
    SOMI_REQUIRE(logits && temperature && uniform && out, "sample_no_alloc: a null pointer among the arguments");
    const int64_t need = (int64_t)rows * ceil_div(vocab, SAMPLE_CHUNK) * 3;
    SOMI_REQUIRE(need <= SOMI_SAMPLE_SCRATCH_FLOATS,
                 "sample_no_alloc: %d rows of %d logits need %lld floats of workspace, the fixed one holds %d "
                 "(rows * ceil(vocab / %d) * 3 must not exceed it); use somi_sample with a workspace of your own",
                 rows, vocab, (long long)need, SOMI_SAMPLE_SCRATCH_FLOATS, SAMPLE_CHUNK);
    float* workspace = nullptr;
    if (scratch_on_current_device(&workspace) != 0) return 1;
    // every (row, chunk) triple that the second kernel reads is written by the first: nothing to clear
    return somi_sample(logits, rows, vocab, temperature, uniform, out, workspace, stream);
}

// logits[row, id] = logit > 0 ? logit / penalty : logit * penalty for each listed id (ids must be distinct).
__global__ void __launch_bounds__(256)
penalty_kernel(float* __restrict__ logits, int vocab, const int* __restrict__ ids, int n_ids, float penalty) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_ids) return;
    const int id = ids[i];
    if (id < 0 || id >= vocab) return;
    const float v = logits[id];
    logits[id] = v > 0.f ? v / penalty : v * penalty;
}

extern "C" int somi_repetition_penalty(float* logits_row, int vocab, const int* ids, int n_ids, float penalty,
                                       hipStream_t stream) {
    SOMI_REQUIRE(vocab > 0 && n_ids >= 0, "repetition_penalty: bad sizes");
    SOMI_REQUIRE(penalty > 0.f, "repetition_penalty: penalty must be > 0, got %g", (double)penalty);
    if (n_ids == 0) return 0;
    hipLaunchKernelGGL(penalty_kernel, dim3(ceil_div(n_ids, 256)), dim3(256), 0, stream, logits_row, vocab, ids,
                       n_ids, penalty);
    SOMI_LAUNCH_CHECK("repetition_penalty");
    return 0;
}

// The same rule for several rows at once: the ids of row r are ids[offsets[r] .. offsets[r + 1]) (distinct within a
// row), its penalty penalties[r]; a row with penalty 1 or no ids is left as it is.
__global__ void __launch_bounds__(256)
penalty_rows_kernel(float* __restrict__ logits, int vocab, const int* __restrict__ offsets,
                    const int* __restrict__ ids, const float* __restrict__ penalties) {
    const int row = blockIdx.y;
    const int begin = offsets[row], count = offsets[row + 1] - begin;
    const float penalty = penalties[row];
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count || penalty == 1.0f) return;
    const int id = ids[begin + i];
    if (id < 0 || id >= vocab) return;
    float* at = logits + (int64_t)row * vocab + id;
    const float v = *at;
    *at = v > 0.f ? v / penalty : v * penalty;
}

// logits: [rows, vocab] float32, in place; offsets: [rows + 1] int32 (ascending from 0); ids: [offsets[rows]] int32;
// penalties: [rows] float32, each > 0 (checked by the caller, who holds them on the host); most_ids: the largest
// number of ids a row has.
extern "C" int somi_repetition_penalty_rows(float* logits, int rows, int vocab, const int* offsets, const int* ids,
                                            const float* penalties, int most_ids, hipStream_t stream) {
    SOMI_REQUIRE(rows >= 0 && vocab > 0 && most_ids >= 0, "repetition_penalty_rows: bad sizes");
    SOMI_REQUIRE(rows <= 65535, "repetition_penalty_rows: too many rows");
    if (rows == 0 || most_ids == 0) return 0;
    hipLaunchKernelGGL(penalty_rows_kernel, dim3(ceil_div(most_ids, 256), rows), dim3(256), 0, stream, logits, vocab,
                       offsets, ids, penalties);
    SOMI_LAUNCH_CHECK("repetition_penalty_rows");
    return 0;
}

// ---------------------------------------------------------------------------------------------------------
// Top-k and top-p masks (somi_inference/core/sampler.py:116-157), without sorting the row.
//
// Both rules keep a prefix of the row in descending order: top-k the first k entries; top-p, on softmax(z / T)
// of what top-k left, every entry whose predecessors hold a mass of at most p (so the entry that crosses p
// stays and the first entry is never removed, sampler.py:150-153).  With a weight per entry (1 for top-k,
// the entry's softmax mass for top-p) both are the same search: the entry at which the running weight first
// exceeds a target (k - 1, or p times the total).  One workgroup per row finds that entry's value by a radix
// descent over the 32 bits of an order-preserving key, eight bits at a time: a 256-bin histogram of the
// weights of the entries that match the bits found so far, then the bin in which the running weight crosses.
// Weights are integers (softmax mass in units of 2^-40 of the largest entry's), so sums do not depend on the
// order of the atomic additions and a row's result does not depend on timing or on the batch.  Entries equal
// to the value found are kept in index order, as many as fit; everything below becomes -inf.
#define FILTER_NT 1024
#define FILTER_WAVES (FILTER_NT / 64)
#define FILTER_AHEAD 8
typedef unsigned long long filter_u64;

struct FilterCut {
    unsigned key;        // entries with a larger key stay
    unsigned ties;       // and the first `ties` entries (in index order) with this key
    bool all;            // the target lies beyond the total: everything stays
};

// value order == unsigned order of the key
__device__ __forceinline__ unsigned filter_key(float v) {
    const unsigned bits = __float_as_uint(v);
    return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}
__device__ __forceinline__ float filter_value(unsigned key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}
__device__ __forceinline__ filter_u64 filter_mass(float v, float temp, float zmax) {
    return (filter_u64)(expf(v / temp - zmax) * 1099511627776.0f);           // 2^40; expf(-inf) = 0
}
// The histogram is held FILTER_COPIES times over, a lane adding to copy (lane % FILTER_COPIES): the values of a row
// share their leading bits, so that without copies most lanes of a wavefront would add to one address in turn.
// The copies of a bin lie in different banks.
#define FILTER_COPIES 16

struct FilterShared {
    filter_u64 hist[256 * FILTER_COPIES];
    filter_u64 above, target, group;
    int bin;
    unsigned wave_count[FILTER_WAVES];
    float red[16];
};

// MASS: weights are softmax masses and the target is top_p times their total; else weights are 1 and the target is
// `count_target`.  Called by the whole workgroup; every thread returns the same cut.
template <bool MASS>
__device__ FilterCut filter_select(const float* __restrict__ row, int vocab, float temp, float zmax,
                                   filter_u64 count_target, float top_p, FilterShared& sh) {
    const int tid = threadIdx.x;
    unsigned prefix = 0;
    filter_u64 above = 0, target = count_target, group = 0;
    for (int level = 0; level < 4; ++level) {
        const int shift = 24 - 8 * level;
        for (int b = tid; b < 256 * FILTER_COPIES; b += FILTER_NT) sh.hist[b] = 0;
        __syncthreads();
        for (int base = 0; base < vocab; base += FILTER_AHEAD * FILTER_NT) {
            float v[FILTER_AHEAD];                              // several loads under way before the first is used
#pragma unroll
            for (int a = 0; a < FILTER_AHEAD; ++a) {
                const int i = base + a * FILTER_NT + tid;
                v[a] = i < vocab ? row[i] : 0.f;
            }
#pragma unroll
            for (int a = 0; a < FILTER_AHEAD; ++a) {
                const bool valid = base + a * FILTER_NT + tid < vocab;
                const unsigned key = filter_key(v[a]);
                const bool in = valid && (level == 0 || (key >> (shift + 8)) == (prefix >> (shift + 8)));
                filter_u64 w = 0;
                if (in) w = MASS ? filter_mass(v[a], temp, zmax) : 1ull;
                if (w != 0) atomicAdd(&sh.hist[((key >> shift) & 255u) * FILTER_COPIES + (tid & (FILTER_COPIES - 1))], w);
            }
        }
        __syncthreads();
        if (tid < 64) {
            // lane l holds the bins 255 - 4 l .. 252 - 4 l: descending values in ascending lanes
            filter_u64 local[4], mine = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                local[j] = 0;
#pragma unroll
                for (int c = 0; c < FILTER_COPIES; ++c) local[j] += sh.hist[(255 - 4 * tid - j) * FILTER_COPIES + c];
                mine += local[j];
            }
            filter_u64 incl = mine;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const filter_u64 other = __shfl_up(incl, off, 64);
                if (tid >= off) incl += other;
            }
            if (MASS && level == 0) {
                const filter_u64 total = __shfl(incl, 63, 64);
                target = (filter_u64)((double)top_p * (double)total);
            }
            filter_u64 run = above + incl - mine, found_above = 0;
            filter_u64 found_group = 0;
            int found = -1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (found < 0 && run + local[j] > target) {
                    found = 255 - 4 * tid - j;
                    found_above = run;
                    found_group = local[j];
                }
                run += local[j];
            }
            const filter_u64 finders = __ballot(found >= 0);
            if (finders == 0) {
                if (tid == 0) sh.bin = -1;
            } else if (tid == __ffsll((long long)finders) - 1) {
                sh.bin = found;
                sh.above = found_above;
                sh.target = target;
                sh.group = found_group;
            }
        }
        __syncthreads();
        if (sh.bin < 0) return FilterCut{0u, 0u, true};
        prefix |= (unsigned)sh.bin << shift;
        above = sh.above;
        target = sh.target;
        group = sh.group;
    }
    filter_u64 each = MASS ? filter_mass(filter_value(prefix), temp, zmax) : 1ull;
    if (each == 0) each = 1;
    const filter_u64 members = group / each, fit = (target - above) / each + 1;
    return FilterCut{prefix, (unsigned)(fit < members ? fit : members), false};
}

// Writes -inf over what the cut removes.  Every wavefront walks a contiguous piece of the row, so that "the first
// entries with the key" is a count over the wavefronts before it plus a count over the lanes before it.
__device__ void filter_apply(float* __restrict__ row, int vocab, const FilterCut& cut, FilterShared& sh) {
    if (cut.all) return;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int piece = ((vocab + FILTER_WAVES - 1) / FILTER_WAVES + 63) / 64 * 64;
    const int begin = wave * piece, end = min(vocab, begin + piece);
    unsigned equal = 0;
    for (int base = begin; base < end; base += FILTER_AHEAD * 64) {
        float v[FILTER_AHEAD];
#pragma unroll
        for (int a = 0; a < FILTER_AHEAD; ++a) {
            const int i = base + a * 64 + lane;
            v[a] = i < end ? row[i] : 0.f;
        }
#pragma unroll
        for (int a = 0; a < FILTER_AHEAD; ++a)
            equal += __popcll(__ballot(base + a * 64 + lane < end && filter_key(v[a]) == cut.key));
    }
    if (lane == 0) sh.wave_count[wave] = equal;
    __syncthreads();
    unsigned before = 0;
    for (int w = 0; w < wave; ++w) before += sh.wave_count[w];
    for (int base = begin; base < end; base += FILTER_AHEAD * 64) {
        float v[FILTER_AHEAD];
#pragma unroll
        for (int a = 0; a < FILTER_AHEAD; ++a) {
            const int i = base + a * 64 + lane;
            v[a] = i < end ? row[i] : 0.f;
        }
#pragma unroll
        for (int a = 0; a < FILTER_AHEAD; ++a) {
            const int i = base + a * 64 + lane;
            const bool valid = i < end;
            const unsigned key = filter_key(v[a]);
            const filter_u64 same = __ballot(valid && key == cut.key);
            const unsigned rank = before + __popcll(same & ((1ull << lane) - 1ull));
            const bool keep = key > cut.key || (key == cut.key && rank < cut.ties);
            if (valid && !keep) row[i] = -INFINITY;
            before += __popcll(same);
        }
    }
    __syncthreads();
}

__global__ void __launch_bounds__(FILTER_NT)
sample_filter_kernel(float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
                     const int* __restrict__ top_k, const float* __restrict__ top_p) {
    __shared__ FilterShared sh;
    float* row = logits + (int64_t)blockIdx.x * vocab;
    const float temp = temperature[blockIdx.x];
    if (!(temp > 0.f)) return;                              // greedy rows skip both rules (sampler.py:123, 142)
    const int k = top_k[blockIdx.x];
    const float p = top_p[blockIdx.x];
    if (k > 0 && k < vocab) {
        const FilterCut cut = filter_select<false>(row, vocab, temp, 0.f, (filter_u64)(k - 1), 0.f, sh);
        filter_apply(row, vocab, cut, sh);
    }
    if (p < 1.0f) {
        float zmax = -INFINITY;
#pragma unroll 8
        for (int i = threadIdx.x; i < vocab; i += FILTER_NT) zmax = fmaxf(zmax, row[i] / temp);
        zmax = block_max<FILTER_NT>(zmax, sh.red);
        if (zmax == -INFINITY) return;
        const FilterCut cut = filter_select<true>(row, vocab, temp, zmax, 0, p, sh);
        filter_apply(row, vocab, cut, sh);
    }
}

// logits: [rows, vocab] float32, in place; temperature, top_p: [rows] float32; top_k: [rows] int32 (-1 or >= vocab:
// off).  Rows with temperature 0 are left as they are.
extern "C" int somi_sample_filter(float* logits, int rows, int vocab, const float* temperature, const int* top_k,
                                  const float* top_p, hipStream_t stream) {
    SOMI_REQUIRE(rows >= 0 && vocab > 0, "sample_filter: bad sizes rows=%d vocab=%d", rows, vocab);
    SOMI_REQUIRE(vocab <= (1 << 22), "sample_filter: vocabulary of %d is beyond the 2^22 that the integer masses hold", vocab);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(sample_filter_kernel, dim3(rows), dim3(FILTER_NT), 0, stream, logits, vocab, temperature, top_k,
                       top_p);
    SOMI_LAUNCH_CHECK("sample_filter");
    return 0;
}
