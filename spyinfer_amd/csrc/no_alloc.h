// Entry points of the kernel library that allocate nothing.
//
// They have no counterpart in the reference.  They are for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// Such a caller still brings the inputs and outputs; what the kernels need beyond them (partial
// results of the first kernel for the second) lies in an array of fixed size inside the library,
// one copy per GPU, held until the process ends.
#pragma once
#include <hip/hip_runtime.h>

// Most rows (R) that spy_sample_static takes.  Its scratch array holds 3 * 64 floats per row:
// 384 KiB per GPU at this limit.
#define SPY_SAMPLE_STATIC_MAX_ROWS 512

// spy_sample with its workspace inside the library: out[r] = first maximum of logits[r] if
// temperature[r] == 0, else the token at which the cumulative probability of
// softmax(logits[r] / temperature[r]), over ascending ids, first exceeds uniform[r].
// Same kernels and same results as spy_sample.  Calls no hipMalloc, hipFree or other allocating
// routine.  R > SPY_SAMPLE_STATIC_MAX_ROWS is refused (returns 1, spy_last_error() says why).
// Every call on a GPU uses that GPU's one scratch array, which keeps the last call's contents;
// the kernels write every element before they read it, so nothing has to be cleared.  Calls that
// overlap on one GPU (two streams, two threads) race on it: a caller must order them.
extern "C" int spy_sample_static(const float* logits, const float* temperature, const float* uniform, int* out, int R, int V,
                                 hipStream_t st);
