// Token choice from float32 logits: greedy argmax, or a draw from softmax(logits / T).
//
// Reference: somi_inference/core/sampler.py:104-114 (logits /= T when T > 0), :159-176 (T == 0: argmax,
// else float32 softmax and one multinomial draw) and :80-102 (repetition penalty: a positive logit is
// divided by the penalty, a non-positive one multiplied).  The draw here is by inverse CDF from a uniform
// number that the host derives from the request's own seed and token count, so a request's tokens do not
// depend on what else is in the batch.
#include "common.h"

#define SAMPLE_NT 1024

__global__ void __launch_bounds__(SAMPLE_NT)
sample_kernel(const float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
              const float* __restrict__ uniform, int* __restrict__ out) {
    __shared__ float red[16];
    __shared__ float part[SAMPLE_NT];
    __shared__ int idxs[SAMPLE_NT];
    __shared__ float s_target;
    __shared__ int s_owner;
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* z = logits + (int64_t)row * vocab;
    const float temp = temperature[row];
    const int chunk = (vocab + SAMPLE_NT - 1) / SAMPLE_NT;
    const int begin = tid * chunk < vocab ? tid * chunk : vocab;
    const int end = begin + chunk < vocab ? begin + chunk : vocab;

    if (temp == 0.f) {
        // first index of the maximum (torch.argmax on ties is not specified; the first is the rule here)
        float best = -INFINITY;
        int best_i = vocab;
        for (int i = begin; i < end; ++i) {
            const float v = z[i];
            if (v > best || best_i == vocab) { best = v; best_i = i; }
        }
        part[tid] = best;
        idxs[tid] = best_i;
        __syncthreads();
        for (int step = SAMPLE_NT / 2; step > 0; step >>= 1) {
            if (tid < step) {
                const float ov = part[tid + step];
                const int oi = idxs[tid + step];
                const bool take = oi < vocab && (idxs[tid] == vocab || ov > part[tid] ||
                                                 (ov == part[tid] && oi < idxs[tid]));
                if (take) { part[tid] = ov; idxs[tid] = oi; }
            }
            __syncthreads();
        }
        if (tid == 0) out[row] = idxs[0];
        return;
    }

    float mx = -INFINITY;
    for (int i = begin; i < end; ++i) mx = fmaxf(mx, z[i] / temp);
    mx = block_max<SAMPLE_NT>(mx, red);
    float sum = 0.f;
    for (int i = begin; i < end; ++i) sum += expf(z[i] / temp - mx);
    part[tid] = sum;
    __syncthreads();
    if (tid == 0) {
        // exclusive prefix of the per-thread masses, in index order
        float run = 0.f;
        int owner = -1, last_nonzero = 0;
        for (int k = 0; k < SAMPLE_NT; ++k) {
            const float mass = part[k];
            part[k] = run;
            if (mass > 0.f) last_nonzero = k;
            run += mass;
        }
        const float target = uniform[row] * run;
        for (int k = 0; k < SAMPLE_NT; ++k) {
            const float hi = (k + 1 < SAMPLE_NT) ? part[k + 1] : run;
            if (target >= part[k] && target < hi) { owner = k; break; }
        }
        s_owner = owner < 0 ? last_nonzero : owner;
        s_target = target;
    }
    __syncthreads();
    if (tid == s_owner) {
        float run = part[tid];
        int pick = -1, last = begin;
        for (int i = begin; i < end; ++i) {
            const float w = expf(z[i] / temp - mx);
            if (w > 0.f) last = i;
            run += w;
            if (run > s_target) { pick = i; break; }
        }
        out[row] = pick < 0 ? last : pick;
    }
}

// logits: [rows, vocab] float32; temperature, uniform: [rows] float32 (uniform in [0, 1)); out: [rows] int32.
extern "C" int somi_sample(const float* logits, int rows, int vocab, const float* temperature,
                           const float* uniform, int* out, hipStream_t stream) {
    SOMI_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_NT), 0, stream, logits, vocab, temperature, uniform,
                       out);
    SOMI_LAUNCH_CHECK("sample");
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
