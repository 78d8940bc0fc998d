// The one entry point of these libraries that allocates nothing and takes no workspace.
//
// It has no counterpart in the reference.  It is there for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// Partial maxima the fixed array holds: rows x ceil(vocab / 4096) of a call may not exceed it
// (64 rows of a 262144-token vocabulary; 32 KB of device memory on every GPU the library runs on,
// held until the process ends).
#define SE_NO_ALLOC_SAMPLE_SLOTS 4096

// se_sample_unfiltered (sampling.hip) without its workspace arguments: one token per row of float
// `logits [rows, vocab]` (row stride `stride`), the arg-max for rows whose temperature is absent
// or 0, else the arg-max of logit / temperature + Gumbel noise keyed by the row's seed; `temperature`
// and `seeds` may be null.  Returns 0, -1 for sizes beyond the limit above (nothing is launched),
// -2 if the array's address cannot be had or a launch fails.  It calls no allocating routine.
// All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (other
// streams, other threads) race; calls on one stream do not.
extern "C" int se_sample_unfiltered_no_alloc(const float* logits, int64_t stride, int rows, int vocab,
                                             const float* temperature, const uint64_t* seeds,
                                             int32_t* out, hipStream_t stream);
