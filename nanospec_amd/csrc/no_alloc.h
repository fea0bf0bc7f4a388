// Entry points that allocate nothing.
//
// They have no counterpart in ved1beta/nanospec (whose products are library calls that bring their own workspaces).  They are
// for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc.  Such a caller passes inputs and outputs only; what the kernels need beyond them lies in an array that
// the library itself holds on every GPU it runs on, from the library's load until the process ends.
#pragma once
#include <hip/hip_runtime.h>

// The most 32-bit partial sums the array holds: 8 MiB on each GPU.
#define NS_STATIC_SCRATCH_FLOATS (2u * 1024u * 1024u)

extern "C" {

// Finds the calling thread's current GPU's copy of the array (no allocation; once per GPU, later calls return at once).
// ns_gemm_wide_bf16_static does this by itself at its first call on a GPU; a caller that is going to capture a graph calls
// it beforehand, so that nothing but launches happens under capture.  -> 0, or a HIP error code.
int ns_static_scratch_init(void);

// ns_gemm_wide_bf16 (out[M, N] = x[M, K] . wt[N, K]^T for up to 128 bfloat16 rows from a tiled weight, K cut into `ksplit`
// ranges; epi 1: silu(x . wt^T) * (x . wt2^T)) with the partial sums of the ranges in the library's own array instead of a
// workspace argument.  Arguments as ns_gemm_wide_bf16 without `workspace` and `defer`.
// Refuses with NS_ERR_SCRATCH_TOO_SMALL when (wt2 ? 2 : 1) * ksplit * M * N exceeds NS_STATIC_SCRATCH_FLOATS (a single
// range needs none).  Calls no hipMalloc, hipFree or other allocating routine.
// Every call on a GPU uses that GPU's one array, which keeps the last call's contents.  Nothing in it has to start at
// zero: the first kernel writes every partial sum that the second reads.  Two calls that overlap on one GPU (different
// streams, or different threads) race on it; calls on one stream are ordered and safe.
int ns_gemm_wide_bf16_static(void* out, const void* x, const void* wt, const void* wt2, int M, int N, int K, int x_stride,
                             int out_stride, int epi, int out_f32, int ksplit, int nt, hipStream_t stream);
}
