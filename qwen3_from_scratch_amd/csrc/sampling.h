// The sampling library's entry points.
#pragma once

#include <hip/hip_runtime.h>

// Bytes of the device array that q3_sample_static keeps per GPU: room for 256 rows of a
// vocabulary of 151,936 columns (q3_sample_workspace(256, 151936) = 306,176 bytes).
#define Q3_SAMPLE_STATIC_BYTES (320 * 1024)

extern "C" {

// How many chunks a row of V columns is cut into, and the bytes of workspace q3_sample needs.
int q3_sample_chunks(int V);
long q3_sample_workspace(int R, int V);

// One token per row of float32 logits (R, V): arg-max where temperature[r] <= 0, else a draw
// from softmax(logits / temperature) among the top_k[r] best (all if top_k[r] <= 0), keyed by
// (seed[r], counter[r], column). `workspace`: q3_sample_workspace(R, V) bytes, 8-byte aligned.
int q3_sample(const float* logits, const float* temperature, const int* top_k, const long long* seed,
              const int* counter, int* out, int R, int V, int with_top_k, void* workspace, hipStream_t stream);

// q3_sample without a workspace argument and without any allocation: no hipMalloc, hipFree or
// allocating library call is made, in the first call or later. It has no counterpart in the
// reference; it is for callers that cannot allocate: code under HIP graph capture, tight serving
// loops, harnesses that forbid allocation. The kernels' intermediate results go to a device array
// of Q3_SAMPLE_STATIC_BYTES that the library holds on every GPU it runs on until the process
// ends; a call whose R and V need more (q3_sample_workspace(R, V) > Q3_SAMPLE_STATIC_BYTES) is
// refused with Q3_ERR_UNSUPPORTED (10002) and launches nothing. All calls on one GPU share that
// GPU's array: calls that overlap there (two streams, two threads) race; calls on one stream do
// not. Inputs and outputs are the caller's, as for q3_sample, and the result is the same.
// The first call on a device asks the runtime for the address of that device's array
// (hipGetSymbolAddress, under a lock); make it outside a graph capture. Later calls launch
// kernels only and may be captured.
int q3_sample_static(const float* logits, const float* temperature, const int* top_k, const long long* seed,
                     const int* counter, int* out, int R, int V, int with_top_k, hipStream_t stream);
}
