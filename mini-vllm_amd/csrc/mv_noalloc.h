// An entry point that allocates nothing.
//
// mv_sample_noalloc has no counterpart in the reference (w4096/mini-vllm samples through library
// calls that allocate as they please). It is for callers that cannot allocate device memory: code
// that runs under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// It draws one token per row like mv_sample (same kernels, same results), but the partial results
// that the workgroups sharing a row exchange live in a device array that is part of the library
// (file scope, static, MV_NOALLOC_SCRATCH_BYTES = 256 KiB on every GPU the library runs on, held
// until the process ends) instead of a workspace the caller brings. The caller still passes
// inputs and outputs. Limits: at most MV_NOALLOC_MAX_ROWS rows a call; more are refused with an
// error (mv_last_error()), never computed wrongly. The call makes no hipMalloc, hipFree or other
// allocating call. Nothing in the array has to start at zero: every slot the second pass reads
// was written by the first pass of the same call. All calls on one GPU share that GPU's array:
// calls that overlap in time on one GPU (two streams, two threads) race; calls in stream order do not.
#pragma once

#include <hip/hip_runtime.h>

#define MV_NOALLOC_MAX_ROWS 1024
#define MV_NOALLOC_CHUNKS 32
#define MV_NOALLOC_SCRATCH_BYTES (MV_NOALLOC_MAX_ROWS * MV_NOALLOC_CHUNKS * 8)

// logits float [M, ld >= V]; temperature, top_k, top_p per row or null (0 / off / off); rng
// [M][2] = (seed, counter), needed when temperatures are given; out int32 [M]. Returns 0, or
// non-zero with the reason in mv_last_error().
extern "C" int mv_sample_noalloc(const float* logits, long ld, int M, int V, const float* temperature,
                                 const int* top_k, const float* top_p, const unsigned long long* rng, int* out,
                                 hipStream_t stream);
