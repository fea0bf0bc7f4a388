// out[M, N] = x[M, K] . w[N, K]^T  with 32-bit accumulation in a fixed order, for any M, N, K.
//
// The plain tiled kernel of the true 32-bit path, and the fall-back for shapes the matrix-core
// kernels refuse.  Every output element is one chain of fused multiply-adds over k = 0..K-1, so
// a row's result does not depend on which other rows share the launch.  (Up to 8 rows of 32-bit x go through a
// second kernel below, which reads w as fast as memory gives it; its sums are ordered differently, so a token's
// 32-bit result as one of few rows and as one of many differ by rounding.)
// (reference: the nn.Linear calls of model/llama.py:175,184,195,286)
#include "common.h"

#define GT_M 64
#define GT_N 64
#define GT_K 16

template <typename T, typename OutT>
__global__ __launch_bounds__(256) void gemm_generic_kernel(OutT* __restrict__ out, const T* __restrict__ x,
                                                            const T* __restrict__ w, int M, int N, int K, int x_stride,
                                                            int out_stride) {
  __shared__ float xs[GT_K][GT_M + 4];
  __shared__ float ws[GT_K][GT_N + 4];
  const int m0 = blockIdx.y * GT_M, n0 = blockIdx.x * GT_N;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;  // 16 x 16 threads, 4 x 4 outputs each
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GT_K) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread; k is the fast index of a thread's loads
    for (int e = threadIdx.x; e < GT_M * GT_K; e += 256) {
      const int r = e / GT_K, kk = e % GT_K;
      const int m = m0 + r, n = n0 + r, k = k0 + kk;
      xs[kk][r] = (m < M && k < K) ? to_f(x[(size_t)m * x_stride + k]) : 0.f;
      ws[kk][r] = (n < N && k < K) ? to_f(w[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GT_K; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[(size_t)m * out_stride + n] = (OutT)acc[i][j];
    }
  }
}

// Few rows (decode) in 32-bit: the work is reading w once.  A wave owns ROWS_N rows of w and walks K with 16-byte
// loads, every lane summing its own k (lane, lane + 64, ... in units of four) in order for each of up to ROWS_M rows of
// x; the 64 partial sums of an output are then added by a fixed butterfly.  An output's value depends on its own row of
// x and of w only.  For K and the row strides multiples of 4 and 16-byte aligned operands.
#define ROWS_M 8
#define ROWS_N 4
__global__ __launch_bounds__(256) void gemm_rows_f32_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                            const float* __restrict__ w, int M, int N, int K, int x_stride,
                                                            int out_stride) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * 4 + wave) * ROWS_N;
  if (n0 >= N) return;
  float acc[ROWS_N][ROWS_M];
#pragma unroll
  for (int j = 0; j < ROWS_N; ++j)
#pragma unroll
    for (int m = 0; m < ROWS_M; ++m) acc[j][m] = 0.f;
  const float4* wr[ROWS_N];
#pragma unroll
  for (int j = 0; j < ROWS_N; ++j) wr[j] = reinterpret_cast<const float4*>(w + (size_t)min(n0 + j, N - 1) * K);
  const int k4 = K / 4;
  for (int i = lane; i < k4; i += 64) {
    float4 wv[ROWS_N];
#pragma unroll
    for (int j = 0; j < ROWS_N; ++j) wv[j] = wr[j][i];
#pragma unroll
    for (int m = 0; m < ROWS_M; ++m) {
      if (m < M) {  // uniform
        const float4 xv = reinterpret_cast<const float4*>(x + (size_t)m * x_stride)[i];
#pragma unroll
        for (int j = 0; j < ROWS_N; ++j) {
          float a = acc[j][m];
          a = fmaf(xv.x, wv[j].x, a);
          a = fmaf(xv.y, wv[j].y, a);
          a = fmaf(xv.z, wv[j].z, a);
          a = fmaf(xv.w, wv[j].w, a);
          acc[j][m] = a;
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < ROWS_N; ++j)
#pragma unroll
    for (int m = 0; m < ROWS_M; ++m) {
      if (m < M) {
        float v = acc[j][m];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        if (lane == 0 && n0 + j < N) out[(size_t)m * out_stride + n0 + j] = v;
      }
    }
}

// out_f32 != 0 writes 32-bit results whatever the input type (logits).
extern "C" int ns_gemm_generic(void* out, const void* x, const void* w, int M, int N, int K, int x_stride, int out_stride,
                               int out_f32, int dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || x_stride < K || out_stride < N) return NS_ERR_BAD_ARG;
  dim3 grid((N + GT_N - 1) / GT_N, (M + GT_M - 1) / GT_M);
  if (grid.y > 65535) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32 && M <= ROWS_M && K % 4 == 0 && x_stride % 4 == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0) {
    gemm_rows_f32_kernel<<<(N + 4 * ROWS_N - 1) / (4 * ROWS_N), 256, 0, stream>>>((float*)out, (const float*)x, (const float*)w, M, N, K,
                                                                                  x_stride, out_stride);
    return ns_launch_status();
  }
  if (dtype == NS_DTYPE_F32)
    gemm_generic_kernel<float, float><<<grid, 256, 0, stream>>>((float*)out, (const float*)x, (const float*)w, M, N, K, x_stride, out_stride);
  else if (dtype == NS_DTYPE_BF16 && out_f32)
    gemm_generic_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((float*)out, (const bf16_t*)x, (const bf16_t*)w, M, N, K, x_stride, out_stride);
  else if (dtype == NS_DTYPE_BF16)
    gemm_generic_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)x, (const bf16_t*)w, M, N, K, x_stride, out_stride);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
