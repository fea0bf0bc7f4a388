// Embedding gather, RMS norm (with the residual sum fused in), rotary encoding fused with the
// write of keys and values into cache pages, and SiLU(gate)*up.  One template per kernel over the
// storage type (float or bfloat16); all arithmetic is 32-bit.
#include "common.h"

// ------------------------------------------------------------------------------------------------
// Embedding: out[i, :] = table[ids[i], :]                     (reference: model/llama.py:221)
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(T* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids, int hidden) {
  const int row = blockIdx.x;
  const T* src = table + (size_t)ids[row] * hidden;
  T* dst = out + (size_t)row * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
}

extern "C" int ns_embed(void* out, const void* table, const int* ids, int n_tokens, int hidden, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || hidden <= 0) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    embed_kernel<float><<<n_tokens, 256, 0, stream>>>((float*)out, (const float*)table, ids, hidden);
  else if (dtype == NS_DTYPE_BF16)
    embed_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)table, ids, hidden);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// RMS norm with optional residual sum and optional row gather.
//   r = rows ? rows[i] : i
//   v = resid[r] (+ x[r])                 summed in 32-bit, rounded to T (the stream's precision)
//   if write_resid: resid[r] = v
//   out[i] = w * T(v * rsqrt(mean(v^2) + eps))      -- the cast to T precedes the multiplication by w
// (reference: model/llama.py:92-95 for the norm, :207-208 for the sums; the fused form :247-253)
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void rmsnorm_kernel(T* __restrict__ out, T* resid, const T* __restrict__ x, const T* __restrict__ w,
                               const int* __restrict__ rows, int dim, float eps, int write_resid) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  const T* xr = x ? x + r * dim : nullptr;
  T* rr = resid ? resid + r * dim : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < dim; c += blockDim.x) {
    float v = rr ? to_f(rr[c]) : 0.f;
    if (xr) v += to_f(xr[c]);
    v = round_to<T>(v);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rinv = rsqrtf(ss / (float)dim + eps);
  T* o = out + (size_t)i * dim;
  for (int c = threadIdx.x; c < dim; c += blockDim.x) {
    float v = rr ? to_f(rr[c]) : 0.f;
    if (xr) v += to_f(xr[c]);
    const T vt = from_f<T>(v);
    if (write_resid && rr && xr) rr[c] = vt;
    o[c] = from_f<T>(to_f(w[c]) * round_to<T>(to_f(vt) * rinv));
  }
}

extern "C" int ns_rmsnorm(void* out, void* resid, const void* x, const void* w, const int* rows, int n_rows, int dim,
                          float eps, int write_resid, int dtype, hipStream_t stream) {
  if (n_rows <= 0 || dim <= 0 || (!resid && !x)) return NS_ERR_BAD_ARG;
  if (write_resid && rows) return NS_ERR_BAD_ARG;  // a gathered row may be named twice
  const int threads = dim >= 2048 ? 512 : 256;
  if (dtype == NS_DTYPE_F32)
    rmsnorm_kernel<float><<<n_rows, threads, 0, stream>>>((float*)out, (float*)resid, (const float*)x, (const float*)w, rows, dim, eps, write_resid);
  else if (dtype == NS_DTYPE_BF16)
    rmsnorm_kernel<bf16_t><<<n_rows, threads, 0, stream>>>((bf16_t*)out, (bf16_t*)resid, (const bf16_t*)x, (const bf16_t*)w, rows, dim, eps, write_resid);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// Rotary encoding of q (in place) and k, fused with the write of k and v into their cache pages.
//   qkv row layout: [heads*hd | kv_heads*hd | kv_heads*hd]
//   pair (j, j + rot/2), j < rot/2:  x_j' = x_j cos - x_{j+rot/2} sin ;  x_{j+rot/2}' = x_{j+rot/2} cos + x_j sin
//   angle = position * inv_freq[j], all in 32-bit            (reference: model/llama.py:133-136,150-158)
//   K page layout: [page][token in page][kv head][hd]        (reference: kv/cache.py:16-26)
//   V page layout: [page][kv head][hd][token in page]        (transposed: the attention kernels read 4 or 8
//                                                             consecutive tokens of one channel in one load)
//   page = block_table[req * table_stride + position / page_size]
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void rope_kv_kernel(T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                               const int* __restrict__ token_req, const int* __restrict__ block_table, int table_stride,
                               const float* __restrict__ inv_freq, T* __restrict__ k_cache, T* __restrict__ v_cache,
                               int heads, int kv_heads, int hd, int rot, int page_size, int write_kv) {
  const int t = blockIdx.x;
  const int pos = positions[t];
  T* row = qkv + (size_t)t * row_stride;
  const int half = rot / 2;
  const float fpos = (float)pos;
  // q heads, in place
  for (int e = threadIdx.x; e < heads * half; e += blockDim.x) {
    const int h = e / half, j = e - h * half;
    const float ang = fpos * inv_freq[j];
    const float c = cosf(ang), s = sinf(ang);
    T* p = row + h * hd;
    const float a = to_f(p[j]), b = to_f(p[j + half]);
    p[j] = from_f<T>(a * c - b * s);
    p[j + half] = from_f<T>(b * c + a * s);
  }
  if (!write_kv) return;
  const int page = block_table[(size_t)token_req[t] * table_stride + pos / page_size];
  const int off = pos % page_size;
  const T* krow = row + heads * hd;
  const T* vrow = krow + kv_heads * hd;
  T* kdst = k_cache + ((size_t)page * page_size + off) * kv_heads * hd;
  T* vdst = v_cache + (size_t)page * kv_heads * hd * page_size + off;
  for (int e = threadIdx.x; e < kv_heads * hd; e += blockDim.x) {
    const int h = e / hd, d = e - h * hd;
    float kv;
    if (d < rot) {
      const int j = d < half ? d : d - half;
      const float ang = fpos * inv_freq[j];
      const float c = cosf(ang), s = sinf(ang);
      const float a = to_f(krow[h * hd + j]), b = to_f(krow[h * hd + j + half]);
      kv = d < half ? a * c - b * s : b * c + a * s;
    } else {
      kv = to_f(krow[e]);
    }
    kdst[e] = from_f<T>(kv);
    vdst[(size_t)e * page_size] = vrow[e];
  }
}

extern "C" int ns_rope_kv_write(void* qkv, int row_stride, const int* positions, const int* token_req,
                                const int* block_table, int table_stride, const float* inv_freq, void* k_cache,
                                void* v_cache, int n_tokens, int heads, int kv_heads, int hd, int rot, int page_size,
                                int write_kv, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || heads <= 0 || kv_heads <= 0 || hd <= 0 || rot < 0 || rot > hd || (rot & 1) || page_size <= 0)
    return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    rope_kv_kernel<float><<<n_tokens, 256, 0, stream>>>((float*)qkv, row_stride, positions, token_req, block_table, table_stride,
                                                        inv_freq, (float*)k_cache, (float*)v_cache, heads, kv_heads, hd, rot, page_size, write_kv);
  else if (dtype == NS_DTYPE_BF16)
    rope_kv_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((bf16_t*)qkv, row_stride, positions, token_req, block_table, table_stride,
                                                         inv_freq, (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, hd, rot, page_size, write_kv);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// out[n, i] = silu(gu[n, i]) * gu[n, inter + i]                 (reference: model/llama.py:195)
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int inter, size_t total) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
    const size_t n = e / inter;
    const int i = (int)(e - n * inter);
    const float g = to_f(gu[n * 2 * inter + i]), u = to_f(gu[n * 2 * inter + inter + i]);
    out[e] = from_f<T>(g / (1.f + expf(-g)) * u);
  }
}

extern "C" int ns_silu_mul(void* out, const void* gu, int n_rows, int inter, int dtype, hipStream_t stream) {
  if (n_rows <= 0 || inter <= 0) return NS_ERR_BAD_ARG;
  const size_t total = (size_t)n_rows * inter;
  const int blocks = (int)((total + 255) / 256 < 65536 ? (total + 255) / 256 : 65536);
  if (dtype == NS_DTYPE_F32)
    silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, inter, total);
  else if (dtype == NS_DTYPE_BF16)
    silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, inter, total);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// A fill kernel for 32-bit words: graphs must not hold memset nodes, so buffers that a captured step
// clears are cleared with this.
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = v;
}
extern "C" int ns_fill_u32(void* p, uint32_t value, size_t n_words, hipStream_t stream) {
  if (n_words == 0) return NS_OK;
  const int blocks = (int)((n_words + 255) / 256 < 4096 ? (n_words + 255) / 256 : 4096);
  fill_u32_kernel<<<blocks, 256, 0, stream>>>((uint32_t*)p, value, n_words);
  return ns_launch_status();
}
