// Entry points of the kernel library that allocate nothing.
//
// somi_sample_no_alloc has no counterpart in the reference (its sampler, somi_inference/core/sampler.py,
// allocates freely through torch).  It is for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, and harnesses that forbid hipMalloc.  It is somi_sample with the per-(row,
// chunk) partial results (maximum, first index, softmax mass) kept in a fixed array in device memory that the
// library holds on every GPU it runs on until the process ends, instead of in a workspace the caller brings.
#pragma once

#include <hip/hip_runtime.h>

// Size of the fixed array: 1 MiB on each GPU.  A call needs rows * ceil(vocab / 2048) * 3 floats of it
// (somi_sample_workspace_floats) and is refused with an error if that is more.
#define SOMI_SAMPLE_SCRATCH_FLOATS (256 * 1024)

// logits: [rows, vocab] float32; temperature, uniform: [rows] float32 (uniform in [0, 1)); out: [rows] int32; all
// in device memory of the current device.  out[r] = argmax of row r where temperature[r] == 0, else an inverse-CDF
// draw from softmax(logits[r] / temperature[r]) at uniform[r]: the same kernels and the same result as somi_sample.
// Calls no hipMalloc, hipFree or other allocating routine.  Every call on a GPU uses that GPU's one array, which
// keeps the last call's contents (each call writes every element it later reads, so nothing has to be cleared):
// calls that overlap on one GPU (two streams, two threads) race; calls on one stream, or ordered by events, do not.
// The first call on a GPU asks the runtime for the array's address on that GPU (hipGetSymbolAddress, which may load
// the library's code for that GPU): make it outside stream capture.  Later calls on that GPU only launch the two
// kernels on `stream` and may be captured into a graph.
// Returns 0, or non-zero after storing a message for somi_last_error().
extern "C" int somi_sample_no_alloc(const float* logits, int rows, int vocab, const float* temperature,
                                    const float* uniform, int* out, hipStream_t stream);

// Largest number of floats somi_sample_no_alloc can use (SOMI_SAMPLE_SCRATCH_FLOATS).
extern "C" int somi_sample_no_alloc_capacity();
