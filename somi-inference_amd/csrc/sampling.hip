// Token choice from float32 logits: greedy argmax, or a draw from softmax(logits / T).
//
// Reference: somi_inference/core/sampler.py:104-114 (logits /= T when T > 0), :159-176 (T == 0: argmax,
// else float32 softmax and one multinomial draw) and :80-102 (repetition penalty: a positive logit is
// divided by the penalty, a non-positive one multiplied).  The draw here is by inverse CDF from a uniform
// number that the host derives from the request's own seed and token count, so a request's tokens do not
// depend on what else is in the batch.
#include "common.h"

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
