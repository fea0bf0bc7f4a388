// Shared device helpers of the nanospec_amd kernels (gfx950 / CDNA4, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

#define NS_DTYPE_F32 0
#define NS_DTYPE_BF16 1
#define NS_WAVE 64

// Error codes returned by every extern "C" entry point (0 = launched).
#define NS_OK 0
#define NS_ERR_BAD_ARG 1001
#define NS_ERR_UNSUPPORTED 1002
#define NS_ERR_SCRATCH_TOO_SMALL 1003

template <typename T> __device__ __forceinline__ float to_f(T v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f(float v) { return (T)v; }
// Round a 32-bit value to the storage type and come back: what a store followed by a load does.
template <typename T> __device__ __forceinline__ float round_to(float v) { return (float)(T)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = NS_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, NS_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = NS_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, NS_WAVE));
  return v;
}

// Block-wide reductions for blocks of up to 1024 threads; `scratch` holds >= 16 floats of LDS.
// Every thread gets the result.  The order of the additions is fixed by the thread layout only.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (NS_WAVE - 1), wave = threadIdx.x / NS_WAVE;
  const int nwaves = (blockDim.x + NS_WAVE - 1) / NS_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = 0.f;
  for (int i = 0; i < nwaves; ++i) r += scratch[i];
  return r;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (NS_WAVE - 1), wave = threadIdx.x / NS_WAVE;
  const int nwaves = (blockDim.x + NS_WAVE - 1) / NS_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = -INFINITY;
  for (int i = 0; i < nwaves; ++i) r = fmaxf(r, scratch[i]);
  return r;
}

static inline int ns_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? NS_OK : (int)e;
}
