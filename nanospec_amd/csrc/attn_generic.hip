// Soft-max attention over the paged cache for any head size and either storage type, one query row
// and one head per workgroup.  It is the attention of the true 32-bit path.  Keys are walked in
// fixed chunks of 256 counted from key 0, so a row's result does not depend on how the tokens were
// cut into steps or on what else is in the batch.
//
// Query row i of request b stands at position p = kv_len[b] - q_len[b] + i and sees the keys
// max(0, p - window + 1) .. p  (window == 0: 0 .. p).          (reference: model/attention.py:22-43)
// Query head h reads key/value head h / (heads / kv_heads).    (reference: model/attention.py:33)
// K pages: [page][kv head][token][hd];  V pages: [page][kv head][hd][token].
#include "common.h"

#define AG_THREADS 256

template <typename T>
__global__ __launch_bounds__(AG_THREADS) void attn_generic_kernel(
    T* __restrict__ out, const T* __restrict__ q, int q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int* __restrict__ token_req, const int* __restrict__ positions,
    const int* __restrict__ block_table, int table_stride, int heads, int kv_heads, int hd, int page_size, float scale,
    int window) {
  extern __shared__ float smem[];  // q_s[hd] | p_s[AG_THREADS] | scratch[16]
  float* q_s = smem;
  float* p_s = smem + hd;
  float* scratch = p_s + AG_THREADS;
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (heads / kv_heads);
  const int pos = positions[t];
  const int* table = block_table + (size_t)token_req[t] * table_stride;
  const T* qrow = q + (size_t)t * q_stride + h * hd;
  for (int d = tid; d < hd; d += AG_THREADS) q_s[d] = to_f(qrow[d]) * scale;
  __syncthreads();
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  float m = -INFINITY, l = 0.f, acc = 0.f;  // acc: channel `tid` of the output (tid < hd)
  for (int c0 = (lo / AG_THREADS) * AG_THREADS; c0 <= pos; c0 += AG_THREADS) {
    const int key = c0 + tid;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = table[key / page_size];
      const T* kr = k_cache + (((size_t)page * kv_heads + kvh) * page_size + key % page_size) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(q_s[d], to_f(kr[d]), dot);
      s = dot;
    }
    const float m_new = fmaxf(m, block_max(s, scratch));
    const float p = valid ? expf(s - m_new) : 0.f;
    p_s[tid] = p;
    const float csum = block_sum(p, scratch);  // its barriers also publish p_s
    const float alpha = m == -INFINITY ? 0.f : expf(m - m_new);
    l = l * alpha + csum;
    m = m_new;
    if (tid < hd) {
      acc *= alpha;
      const int hi = min(AG_THREADS, pos - c0 + 1);
      for (int j = max(0, lo - c0); j < hi; ++j) {
        const int kj = c0 + j;
        const int page = table[kj / page_size];
        const T* vp = v_cache + (((size_t)page * kv_heads + kvh) * hd + tid) * page_size + kj % page_size;
        acc = fmaf(p_s[j], to_f(*vp), acc);
      }
    }
    __syncthreads();
  }
  if (tid < hd) out[((size_t)t * heads + h) * hd + tid] = from_f<T>(acc / l);
}

extern "C" int ns_attn_generic(void* out, const void* q, int q_stride, const void* k_cache, const void* v_cache,
                               const int* token_req, const int* positions, const int* block_table, int table_stride,
                               int n_tokens, int heads, int kv_heads, int hd, int page_size, float scale, int window,
                               int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || hd <= 0 || hd > AG_THREADS || page_size <= 0 || window < 0)
    return NS_ERR_BAD_ARG;
  if (heads > 65535) return NS_ERR_BAD_ARG;
  dim3 grid(n_tokens, heads);
  const size_t smem = (size_t)(hd + AG_THREADS + 16) * sizeof(float);
  if (dtype == NS_DTYPE_F32)
    attn_generic_kernel<float><<<grid, AG_THREADS, smem, stream>>>((float*)out, (const float*)q, q_stride, (const float*)k_cache,
        (const float*)v_cache, token_req, positions, block_table, table_stride, heads, kv_heads, hd, page_size, scale, window);
  else if (dtype == NS_DTYPE_BF16)
    attn_generic_kernel<bf16_t><<<grid, AG_THREADS, smem, stream>>>((bf16_t*)out, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache,
        (const bf16_t*)v_cache, token_req, positions, block_table, table_stride, heads, kv_heads, hd, page_size, scale, window);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}
