// Embedding gather, RMS norm (with the residual sum fused in), rotary encoding fused with the
// write of keys and values into cache pages, and SiLU(gate)*up.  One template per kernel over the
// storage type (float or bfloat16); all arithmetic is 32-bit.
#include "common.h"
#include "rope.h"

// ------------------------------------------------------------------------------------------------
// Embedding: out[i, :] = table[ids[i], :] (* scale, rounded once)      (reference: model/llama.py:221; a scale of 1
//                                                                       copies the row as it is)
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(T* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids, int hidden, float scale) {
  const int row = blockIdx.x;
  const T* src = table + (size_t)ids[row] * hidden;
  T* dst = out + (size_t)row * hidden;
  if (scale == 1.f)
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
  else
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = from_f<T>(to_f(src[i]) * scale);
}

extern "C" int ns_embed(void* out, const void* table, const int* ids, int n_tokens, int hidden, float scale, int dtype,
                        hipStream_t stream) {
  if (n_tokens <= 0 || hidden <= 0) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_F32)
    embed_kernel<float><<<n_tokens, 256, 0, stream>>>((float*)out, (const float*)table, ids, hidden, scale);
  else if (dtype == NS_DTYPE_BF16)
    embed_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)table, ids, hidden, scale);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// ------------------------------------------------------------------------------------------------
// 32-bit logits in place: l = l * scale; with a cap > 0 then l = cap * tanh(l / cap).  For architectures whose head
// ends in a scale or a soft cap; the Llama head has neither and never launches this.
// ------------------------------------------------------------------------------------------------
__global__ void logit_transform_kernel(float* __restrict__ logits, int vocab, int stride, float scale, float cap) {
  float* row = logits + (size_t)blockIdx.y * stride;
  const float inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < vocab; i += gridDim.x * blockDim.x) {
    float v = row[i] * scale;
    if (cap > 0.f) v = cap * tanhf(v * inv_cap);
    row[i] = v;
  }
}

extern "C" int ns_logit_transform(float* logits, int rows, int vocab, int stride, float scale, float cap, hipStream_t stream) {
  if (rows <= 0 || rows > 65535 || vocab <= 0 || stride < vocab || cap < 0.f) return NS_ERR_BAD_ARG;
  const int bx = (vocab + 1023) / 1024 < 64 ? (vocab + 1023) / 1024 : 64;
  logit_transform_kernel<<<dim3(bx, rows), 256, 0, stream>>>(logits, vocab, stride, scale, cap);
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

// The same with 16-byte accesses and the row kept in registers between the two passes; for rows of a multiple
// of 16 bytes and at most 4 pieces per thread.
template <typename T, int MAXC>
__global__ void rmsnorm_vec_kernel(T* __restrict__ out, T* resid, const T* __restrict__ x, const T* __restrict__ w,
                                   const int* __restrict__ rows, int dim, float eps, int write_resid) {
  constexpr int V = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  const vec_t* xr = x ? reinterpret_cast<const vec_t*>(x + r * dim) : nullptr;
  vec_t* rr = resid ? reinterpret_cast<vec_t*>(resid + r * dim) : nullptr;
  const int nvec = dim / V;
  vec_t val[MAXC];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int idx = threadIdx.x + c * blockDim.x;
    if (idx < nvec) {
      vec_t a = rr ? rr[idx] : vec_t{};
      if (xr) {
        const vec_t b = xr[idx];
        if (rr) {
#pragma unroll
          for (int e = 0; e < V; ++e) a[e] = from_f<T>(to_f(a[e]) + to_f(b[e]));
        } else {
          a = b;
        }
      }
      val[c] = a;
#pragma unroll
      for (int e = 0; e < V; ++e) ss += to_f(a[e]) * to_f(a[e]);
    }
  }
  ss = block_sum(ss, scratch);
  const float rinv = rsqrtf(ss / (float)dim + eps);
  vec_t* o = reinterpret_cast<vec_t*>(out + (size_t)i * dim);
  const vec_t* wv = reinterpret_cast<const vec_t*>(w);
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int idx = threadIdx.x + c * blockDim.x;
    if (idx < nvec) {
      if (write_resid && rr && xr) rr[idx] = val[c];
      const vec_t ww = wv[idx];
      vec_t y;
#pragma unroll
      for (int e = 0; e < V; ++e) y[e] = from_f<T>(to_f(ww[e]) * round_to<T>(to_f(val[c][e]) * rinv));
      o[idx] = y;
    }
  }
}

template <typename T>
static bool launch_rmsnorm_vec(void* out, void* resid, const void* x, const void* w, const int* rows, int n_rows, int dim,
                               float eps, int write_resid, hipStream_t stream) {
  constexpr int V = 16 / sizeof(T);
  if (dim % V) return false;
  if (((uintptr_t)out | (uintptr_t)resid | (uintptr_t)x | (uintptr_t)w) & 15) return false;
  const int nvec = dim / V;
  int threads = ((nvec + 63) / 64) * 64;
  if (threads > 1024) threads = 1024;
  const int chunks = (nvec + threads - 1) / threads;
  if (chunks > 4) return false;
  if (chunks <= 1)
    rmsnorm_vec_kernel<T, 1><<<n_rows, threads, 0, stream>>>((T*)out, (T*)resid, (const T*)x, (const T*)w, rows, dim, eps, write_resid);
  else if (chunks == 2)
    rmsnorm_vec_kernel<T, 2><<<n_rows, threads, 0, stream>>>((T*)out, (T*)resid, (const T*)x, (const T*)w, rows, dim, eps, write_resid);
  else
    rmsnorm_vec_kernel<T, 4><<<n_rows, threads, 0, stream>>>((T*)out, (T*)resid, (const T*)x, (const T*)w, rows, dim, eps, write_resid);
  return true;
}

// The same where x has not been added up yet: x[r][c] = T(sum_s partial[s][r][c]), the ranges of a product whose K was
// cut (gemm_wide.hip), added in order.  One workgroup per row; the row stays in registers between the two passes.
// For dim a multiple of 4 and at most 4 * MAXC * threads.
template <typename T, int MAXC>
__global__ void rmsnorm_partial_kernel(T* __restrict__ out, T* resid, const float* __restrict__ partial, size_t plane, int ksplit,
                                       const T* __restrict__ w, const int* __restrict__ rows, int dim, float eps, int write_resid) {
  typedef T vec4_t __attribute__((ext_vector_type(4)));
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const size_t r = rows ? (size_t)rows[i] : (size_t)i;
  const float4* pr = reinterpret_cast<const float4*>(partial + r * dim);
  const size_t plane4 = plane / 4;
  T* rr = resid ? resid + r * dim : nullptr;
  const int n4 = dim / 4;
  float val[MAXC][4];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int idx = threadIdx.x + c * blockDim.x;
    if (idx < n4) {
      float4 s = pr[idx];
      int k = 1;
      for (; k + 3 < ksplit; k += 4) {  // four ranges' loads in flight, added in order
        float4 t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) t[u] = pr[(size_t)(k + u) * plane4 + idx];
#pragma unroll
        for (int u = 0; u < 4; ++u) { s.x += t[u].x; s.y += t[u].y; s.z += t[u].z; s.w += t[u].w; }
      }
      for (; k < ksplit; ++k) {
        const float4 t = pr[(size_t)k * plane4 + idx];
        s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
      }
      const float xs[4] = {s.x, s.y, s.z, s.w};
      vec4_t rv = {};
      if (rr) rv = *reinterpret_cast<const vec4_t*>(rr + idx * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = round_to<T>(xs[e]);
        if (rr) v = round_to<T>(to_f(rv[e]) + v);
        val[c][e] = v;
        ss += v * v;
      }
    }
  }
  ss = block_sum(ss, scratch);
  const float rinv = rsqrtf(ss / (float)dim + eps);
  T* o = out + (size_t)i * dim;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int idx = threadIdx.x + c * blockDim.x;
    if (idx < n4) {
      const vec4_t wv = *reinterpret_cast<const vec4_t*>(w + idx * 4);
      vec4_t rv, ov;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        rv[e] = from_f<T>(val[c][e]);
        ov[e] = from_f<T>(to_f(wv[e]) * round_to<T>(val[c][e] * rinv));
      }
      if (write_resid && rr) *reinterpret_cast<vec4_t*>(rr + idx * 4) = rv;
      *reinterpret_cast<vec4_t*>(o + idx * 4) = ov;
    }
  }
}

// partial: float32 [ksplit][plane / dim rows][dim].
extern "C" int ns_rmsnorm_partial(void* out, void* resid, const void* partial, size_t plane, int ksplit, const void* w,
                                  const int* rows, int n_rows, int dim, float eps, int write_resid, int dtype,
                                  hipStream_t stream) {
  if (n_rows <= 0 || dim <= 0 || (dim & 3) || ksplit < 1 || !partial || (plane & 3) || ((uintptr_t)partial & 15) ||
      (((uintptr_t)out | (uintptr_t)resid | (uintptr_t)w) & 7))
    return NS_ERR_BAD_ARG;
  if (write_resid && rows) return NS_ERR_BAD_ARG;
  if (dtype != NS_DTYPE_BF16) return NS_ERR_UNSUPPORTED;
  const int n4 = dim / 4;
  const int threads = n4 <= 256 ? 256 : n4 <= 2048 ? 512 : 1024;
  const int chunks = (n4 + threads - 1) / threads;
  if (chunks > 4) return NS_ERR_UNSUPPORTED;
  if (chunks <= 1)
    rmsnorm_partial_kernel<bf16_t, 1><<<n_rows, threads, 0, stream>>>((bf16_t*)out, (bf16_t*)resid, (const float*)partial, plane, ksplit, (const bf16_t*)w, rows, dim, eps, write_resid);
  else if (chunks == 2)
    rmsnorm_partial_kernel<bf16_t, 2><<<n_rows, threads, 0, stream>>>((bf16_t*)out, (bf16_t*)resid, (const float*)partial, plane, ksplit, (const bf16_t*)w, rows, dim, eps, write_resid);
  else
    rmsnorm_partial_kernel<bf16_t, 4><<<n_rows, threads, 0, stream>>>((bf16_t*)out, (bf16_t*)resid, (const float*)partial, plane, ksplit, (const bf16_t*)w, rows, dim, eps, write_resid);
  return ns_launch_status();
}

extern "C" int ns_rmsnorm(void* out, void* resid, const void* x, const void* w, const int* rows, int n_rows, int dim,
                          float eps, int write_resid, int dtype, hipStream_t stream) {
  if (n_rows <= 0 || dim <= 0 || (!resid && !x)) return NS_ERR_BAD_ARG;
  if (write_resid && rows) return NS_ERR_BAD_ARG;  // a gathered row may be named twice
  const int threads = dim >= 2048 ? 512 : 256;
  if (dtype == NS_DTYPE_F32 && launch_rmsnorm_vec<float>(out, resid, x, w, rows, n_rows, dim, eps, write_resid, stream)) return ns_launch_status();
  if (dtype == NS_DTYPE_BF16 && launch_rmsnorm_vec<bf16_t>(out, resid, x, w, rows, n_rows, dim, eps, write_resid, stream)) return ns_launch_status();
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
//   K page layout: [page][kv head][token in page][hd]        (the reference keeps [page][token][kv head][hd],
//                                                             kv/cache.py:16-26; here a head's keys of a page are
//                                                             contiguous, which is how the attention kernels read them)
//   V page layout: [page][kv head][hd][token in page]        (transposed: the attention kernels read 4 or 8
//                                                             consecutive tokens of one channel in one load)
//   page = block_table[req * table_stride + position / page_size]
// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ void rope_kv_kernel(T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                               const int* __restrict__ token_req, const int* __restrict__ block_table, int table_stride,
                               const float* __restrict__ inv_freq, T* __restrict__ k_cache, T* __restrict__ v_cache,
                               int heads, int kv_heads, int hd, RopeForm form, int page_size, int write_kv) {
  extern __shared__ float cs[];  // cos[half] | sin[half] of this token's angles
  const int t = blockIdx.x;
  const int pos = positions[t];
  T* row = qkv + (size_t)t * row_stride;
  const int rot = form.rot, half = rot / 2;
  for (int j = threadIdx.x; j < half; j += blockDim.x) rope_cos_sin(form, pos, inv_freq[j], cs[j], cs[half + j]);
  __syncthreads();
  // q heads, in place
  for (int e = threadIdx.x; e < heads * half; e += blockDim.x) {
    const int h = e / half, j = e - h * half;
    int d1, d2;
    rope_pair_channels(form, j, d1, d2);
    T* p = row + h * hd;
    float a, b;
    rope_turn(to_f(p[d1]), to_f(p[d2]), cs[j], cs[half + j], a, b);
    p[d1] = from_f<T>(a);
    p[d2] = from_f<T>(b);
  }
  if (!write_kv) return;
  const int page = block_table[(size_t)token_req[t] * table_stride + pos / page_size];
  const int off = pos % page_size;
  const T* krow = row + heads * hd;
  const T* vrow = krow + kv_heads * hd;
  T* kdst = k_cache + (size_t)page * kv_heads * page_size * hd + (size_t)off * hd;
  T* vdst = v_cache + (size_t)page * kv_heads * hd * page_size + off;
  for (int e = threadIdx.x; e < kv_heads * half; e += blockDim.x) {  // the rotary pairs of k
    const int h = e / half, j = e - h * half;
    int d1, d2;
    rope_pair_channels(form, j, d1, d2);
    float a, b;
    rope_turn(to_f(krow[h * hd + d1]), to_f(krow[h * hd + d2]), cs[j], cs[half + j], a, b);
    kdst[(size_t)h * page_size * hd + d1] = from_f<T>(a);
    kdst[(size_t)h * page_size * hd + d2] = from_f<T>(b);
  }
  const int plain = hd - rot;  // channels of a head beyond the rotary part
  for (int e = threadIdx.x; e < kv_heads * plain; e += blockDim.x) {
    const int h = e / plain, d = rot + e - h * plain;
    kdst[(size_t)h * page_size * hd + d] = krow[h * hd + d];
  }
  for (int e = threadIdx.x; e < kv_heads * hd; e += blockDim.x) vdst[(size_t)e * page_size] = vrow[e];
}

// The same with 16-byte accesses for q and k (values still go element by element into their transposed page): a
// thread takes V consecutive channels j.. of the first half and their partners j + rot/2.  For the half-split pairing,
// rot/2, hd - rot and the row stride multiples of V elements and 16-byte aligned buffers.
template <typename T>
__global__ void rope_kv_vec_kernel(T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                                   const int* __restrict__ token_req, const int* __restrict__ block_table, int table_stride,
                                   const float* __restrict__ inv_freq, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                   int heads, int kv_heads, int hd, RopeForm form, int page_size, int write_kv) {
  constexpr int V = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  extern __shared__ float cs[];  // cos[half] | sin[half] of this token's angles
  const int t = blockIdx.x;
  const int pos = positions[t];
  T* row = qkv + (size_t)t * row_stride;
  const int rot = form.rot, half = rot / 2;
  for (int j = threadIdx.x; j < half; j += blockDim.x) rope_cos_sin(form, pos, inv_freq[j], cs[j], cs[half + j]);
  __syncthreads();
  const int per_head = half / V;  // vector pairs per head
  auto turn = [&](const vec_t a, const vec_t b, int j, vec_t& lo, vec_t& hi) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float x, y;
      rope_turn(to_f(a[e]), to_f(b[e]), cs[j + e], cs[half + j + e], x, y);
      lo[e] = from_f<T>(x);
      hi[e] = from_f<T>(y);
    }
  };
  for (int u = threadIdx.x; u < heads * per_head; u += blockDim.x) {
    const int h = u / per_head, j = (u - h * per_head) * V;
    T* p = row + h * hd + j;
    vec_t lo, hi;
    turn(*reinterpret_cast<const vec_t*>(p), *reinterpret_cast<const vec_t*>(p + half), j, lo, hi);
    *reinterpret_cast<vec_t*>(p) = lo;
    *reinterpret_cast<vec_t*>(p + half) = hi;
  }
  if (!write_kv) return;
  const int page = block_table[(size_t)token_req[t] * table_stride + pos / page_size];
  const int off = pos % page_size;
  const T* krow = row + heads * hd;
  const T* vrow = krow + kv_heads * hd;
  T* kdst = k_cache + (size_t)page * kv_heads * page_size * hd + (size_t)off * hd;
  T* vdst = v_cache + (size_t)page * kv_heads * hd * page_size + off;
  for (int u = threadIdx.x; u < kv_heads * per_head; u += blockDim.x) {
    const int h = u / per_head, j = (u - h * per_head) * V;
    const T* p = krow + h * hd + j;
    vec_t lo, hi;
    turn(*reinterpret_cast<const vec_t*>(p), *reinterpret_cast<const vec_t*>(p + half), j, lo, hi);
    T* d = kdst + (size_t)h * page_size * hd + j;
    *reinterpret_cast<vec_t*>(d) = lo;
    *reinterpret_cast<vec_t*>(d + half) = hi;
  }
  const int plain = (hd - rot) / V;  // vectors of a head beyond the rotary part
  for (int u = threadIdx.x; u < kv_heads * plain; u += blockDim.x) {
    const int h = u / plain, d0 = rot + (u - h * plain) * V;
    *reinterpret_cast<vec_t*>(kdst + (size_t)h * page_size * hd + d0) = *reinterpret_cast<const vec_t*>(krow + h * hd + d0);
  }
  // V pages hold a channel's tokens side by side.  The tokens of a request stand in the batch one after the other at
  // rising positions, so up to V of them fall into one aligned run of V slots of a page: the first of them writes
  // the run for all, a full run as one 16-byte store per channel instead of V stores of one element each.
  const int n_tokens = gridDim.x;
  const int req = token_req[t];
  int cnt = 1;
  if (page_size % V == 0) {
    const bool first = t == 0 || token_req[t - 1] != req;
    if (!first && pos % V != 0) return;  // an earlier token of the run writes this one's values
    const int room = min(V - pos % V, n_tokens - t);
    while (cnt < room && token_req[t + cnt] == req) ++cnt;
  }
  if (cnt == V) {
    for (int e = threadIdx.x; e < kv_heads * hd; e += blockDim.x) {
      vec_t val;
#pragma unroll
      for (int i = 0; i < V; ++i) val[i] = vrow[(size_t)i * row_stride + e];
      *reinterpret_cast<vec_t*>(vdst + (size_t)e * page_size) = val;
    }
  } else {
    for (int e = threadIdx.x; e < kv_heads * hd; e += blockDim.x)
      for (int i = 0; i < cnt; ++i) vdst[(size_t)e * page_size + i] = vrow[(size_t)i * row_stride + e];
  }
}

extern "C" int ns_rope_kv_write(void* qkv, int row_stride, const int* positions, const int* token_req,
                                const int* block_table, int table_stride, const float* inv_freq, void* k_cache,
                                void* v_cache, int n_tokens, int heads, int kv_heads, int hd, int rot, int interleaved,
                                float factor, int page_size, int write_kv, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || heads <= 0 || kv_heads <= 0 || hd <= 0 || rot < 0 || rot > hd || (rot & 1) || page_size <= 0)
    return NS_ERR_BAD_ARG;
  const RopeForm form = {rot, interleaved ? 1 : 0, factor};
  const int work = heads * (rot / 2) > kv_heads * hd ? heads * (rot / 2) : kv_heads * hd;
  const int threads = work >= 1024 ? 1024 : work >= 512 ? 512 : 256;
  const int vlen = dtype == NS_DTYPE_F32 ? 4 : 8;
  const bool aligned = (((uintptr_t)qkv | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0 && row_stride % vlen == 0 && (rot / 2) % vlen == 0 &&
                       (hd - rot) % vlen == 0 && hd % vlen == 0 && rot > 0 && !interleaved;
  if (aligned) {
    const int vthreads = threads >= 512 ? 256 : threads;
    if (dtype == NS_DTYPE_F32)
      rope_kv_vec_kernel<float><<<n_tokens, vthreads, (size_t)(rot + 2) * sizeof(float), stream>>>((float*)qkv, row_stride, positions, token_req, block_table, table_stride,
                                                          inv_freq, (float*)k_cache, (float*)v_cache, heads, kv_heads, hd, form, page_size, write_kv);
    else if (dtype == NS_DTYPE_BF16)
      rope_kv_vec_kernel<bf16_t><<<n_tokens, vthreads, (size_t)(rot + 2) * sizeof(float), stream>>>((bf16_t*)qkv, row_stride, positions, token_req, block_table, table_stride,
                                                           inv_freq, (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, hd, form, page_size, write_kv);
    else
      return NS_ERR_UNSUPPORTED;
    return ns_launch_status();
  }
  if (dtype == NS_DTYPE_F32)
    rope_kv_kernel<float><<<n_tokens, threads, (size_t)(rot + 2) * sizeof(float), stream>>>((float*)qkv, row_stride, positions, token_req, block_table, table_stride,
                                                        inv_freq, (float*)k_cache, (float*)v_cache, heads, kv_heads, hd, form, page_size, write_kv);
  else if (dtype == NS_DTYPE_BF16)
    rope_kv_kernel<bf16_t><<<n_tokens, threads, (size_t)(rot + 2) * sizeof(float), stream>>>((bf16_t*)qkv, row_stride, positions, token_req, block_table, table_stride,
                                                         inv_freq, (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, hd, form, page_size, write_kv);
  else
    return NS_ERR_UNSUPPORTED;
  return ns_launch_status();
}

// The same for a stacked q/k/v product whose K was cut into ranges that are not added up yet (17 to 128 rows through
// ns_gemm_wide_bf16 with `defer`), from the weight tiled in the row order of the fused few-row kernel (gemm_bf16.hip,
// EPI_ROPE_KV): a tile of 16 columns of the product is, in the rotary part of a q or k head, 8 channels j and their
// partners j + rot/2, elsewhere 16 consecutive channels.  One pass adds the ranges in order, rotates the 32-bit sums,
// rounds once, and writes q to the attention input, k to its K page slot and v to the transposed V page.
//   partial[s][m][c]: range s, token m, column c of the product (columns in the tiled row order)
//   thread <-> (token, tile of 16 columns, pair p of columns p and p + 8)
__global__ __launch_bounds__(256) void rope_kv_partial_kernel(bf16_t* __restrict__ q_out, int q_stride, const float* __restrict__ partial,
                                                              int ksplit, int M, int N, const int* __restrict__ positions,
                                                              const int* __restrict__ token_req, const int* __restrict__ block_table,
                                                              int table_stride, const float* __restrict__ inv_freq,
                                                              bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int heads,
                                                              int kv_heads, int hd, RopeForm form, int page_size, int write_kv) {
  const int rot = form.rot;
  const int m = blockIdx.x;
  const int u = blockIdx.y * blockDim.x + threadIdx.x;  // (tile, pair)
  const int tiles_per_head = hd / 16;
  const int tile = u >> 3, p = u & 7;
  if (tile >= (heads + 2 * kv_heads) * tiles_per_head) return;
  const int gh = tile / tiles_per_head, jt = tile - gh * tiles_per_head;  // head among [q heads | k heads | v heads]
  const bool is_q = gh < heads, is_v = gh >= heads + kv_heads;
  if (!is_q && !write_kv) return;
  const int rot_tiles = is_v ? 0 : rot / 16;
  const bool rotary = jt < rot_tiles;
  const size_t plane = (size_t)M * N;
  const float* src = partial + (size_t)m * N + tile * 16 + p;
  float x1 = 0.f, x2 = 0.f;
  for (int s = 0; s < ksplit; ++s) {
    x1 += src[s * plane];
    x2 += src[s * plane + 8];
  }
  const int pos = positions[m];
  int d1, d2;
  if (rotary) {
    const int j = jt * 8 + p;
    float c, sn;
    rope_cos_sin(form, pos, inv_freq[j], c, sn);
    rope_turn(x1, x2, c, sn, x1, x2);
    rope_pair_channels(form, j, d1, d2);
  } else {
    d1 = (is_v ? 0 : rot) + (jt - rot_tiles) * 16 + p;
    d2 = d1 + 8;
  }
  if (is_q) {
    bf16_t* o = q_out + (size_t)m * q_stride + gh * hd;
    o[d1] = (bf16_t)x1;
    o[d2] = (bf16_t)x2;
    return;
  }
  const int page = block_table[(size_t)token_req[m] * table_stride + pos / page_size];
  const int off = pos % page_size;
  if (!is_v) {
    bf16_t* kd = k_cache + (((size_t)page * kv_heads + (gh - heads)) * page_size + off) * hd;
    kd[d1] = (bf16_t)x1;
    kd[d2] = (bf16_t)x2;
  } else {
    bf16_t* vd = v_cache + (((size_t)page * kv_heads + (gh - heads - kv_heads)) * hd) * page_size + off;
    vd[(size_t)d1 * page_size] = (bf16_t)x1;
    vd[(size_t)d2 * page_size] = (bf16_t)x2;
  }
}

extern "C" int ns_rope_kv_partial(void* q_out, int q_stride, const float* partial, int ksplit, int M, int N, const int* positions,
                                  const int* token_req, const int* block_table, int table_stride, const float* inv_freq,
                                  void* k_cache, void* v_cache, int heads, int kv_heads, int hd, int rot, int interleaved,
                                  float factor, int page_size, int write_kv, hipStream_t stream) {
  if (M <= 0 || M > 65535 || ksplit < 1 || heads <= 0 || kv_heads <= 0 || hd <= 0 || (hd & 15) || rot < 0 || rot > hd || (rot & 15) ||
      page_size <= 0 || N != (heads + 2 * kv_heads) * hd || q_stride < heads * hd)
    return NS_ERR_BAD_ARG;
  const int units = N / 2;  // pairs of columns per token
  dim3 grid(M, (units + 255) / 256);
  rope_kv_partial_kernel<<<grid, 256, 0, stream>>>((bf16_t*)q_out, q_stride, partial, ksplit, M, N, positions, token_req, block_table,
                                                   table_stride, inv_freq, (bf16_t*)k_cache, (bf16_t*)v_cache, heads, kv_heads, hd,
                                                   RopeForm{rot, interleaved ? 1 : 0, factor}, page_size, write_kv);
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

template <typename T>
__global__ void silu_mul_vec_kernel(T* __restrict__ out, const T* __restrict__ gu, int inter, size_t total_vec) {
  constexpr int V = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int ivec = inter / V;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total_vec; e += (size_t)gridDim.x * blockDim.x) {
    const size_t n = e / ivec;
    const int i = (int)(e - n * ivec);
    const vec_t g = reinterpret_cast<const vec_t*>(gu + n * 2 * inter)[i];
    const vec_t u = reinterpret_cast<const vec_t*>(gu + n * 2 * inter + inter)[i];
    vec_t y;
#pragma unroll
    for (int k = 0; k < V; ++k) {
      const float gf = to_f(g[k]);
      y[k] = from_f<T>(gf / (1.f + expf(-gf)) * to_f(u[k]));
    }
    reinterpret_cast<vec_t*>(out + n * inter)[i] = y;
  }
}

extern "C" int ns_silu_mul(void* out, const void* gu, int n_rows, int inter, int dtype, hipStream_t stream) {
  if (n_rows <= 0 || inter <= 0) return NS_ERR_BAD_ARG;
  if (dtype == NS_DTYPE_BF16 && inter % 8 == 0 && !(((uintptr_t)out | (uintptr_t)gu) & 15)) {
    const size_t tv = (size_t)n_rows * (inter / 8);
    const int nb = (int)((tv + 255) / 256 < 16384 ? (tv + 255) / 256 : 16384);
    silu_mul_vec_kernel<bf16_t><<<nb, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, inter, tv);
    return ns_launch_status();
  }
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

// A weight matrix back from the layout of the streaming kernels (gemm_bf16.hip:
// wt[rt][kt][i][lane = 16 g + r][e] = w[16 rt + r][128 kt + 32 g + 8 i + e]) into plain rows [N, K], for a library product
// over many rows where only the re-laid copy is kept.  One wave per tile of 16 rows x 128 k: four loads of a contiguous
// kilobyte each; a lane then holds 32 consecutive elements of one row and writes them as 64 contiguous bytes, the four
// lanes of a row 256.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 untile_piece;
// kt0, n_kt: the k tiles to write out (columns 128 kt0 .. of the matrix become columns 0 .. of ``out``).
__global__ __launch_bounds__(256) void untile_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ wt, int N, int K,
                                                     int KT, int kt0, int n_kt, int out_stride, long tiles) {
  const int lane = threadIdx.x & 63;
  const long tile = (long)blockIdx.x * 4 + (threadIdx.x >> 6);  // among the tiles written out
  if (tile >= tiles) return;
  const int rt = (int)(tile / n_kt), kt = kt0 + (int)(tile % n_kt);
  const int r = lane & 15, g = lane >> 4;
  const bf16_t* src = wt + ((size_t)rt * KT + kt) * (16 * 128) + (size_t)lane * 8;
  untile_piece v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = *reinterpret_cast<const untile_piece*>(src + i * 64 * 8);
  const int row = rt * 16 + r;
  if (row >= N) return;
  bf16_t* dst = out + (size_t)row * out_stride + (kt - kt0) * 128 + g * 32;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (kt * 128 + g * 32 + i * 8 < K) *reinterpret_cast<untile_piece*>(dst + i * 8) = v[i];  // K is a multiple of 8
}
// out: bfloat16 [N, columns k0 .. k1 of the matrix] with rows out_stride elements apart, 16-byte aligned; k0 a multiple
// of 128, k1 a multiple of 128 or K; wt: the re-laid matrix (rows padded to 16, k to 128).
extern "C" int ns_untile_bf16(void* out, const void* wt, int N, int K, int k0, int k1, int out_stride, hipStream_t stream) {
  if (N <= 0 || K <= 0 || (K & 7) || (((uintptr_t)out | (uintptr_t)wt) & 15)) return NS_ERR_BAD_ARG;
  if (k0 < 0 || k0 >= k1 || k1 > K || (k0 & 127) || ((k1 & 127) && k1 != K) || out_stride < k1 - k0 || (out_stride & 7)) return NS_ERR_BAD_ARG;
  const int KT = (K + 127) / 128, kt0 = k0 / 128, n_kt = (k1 - k0 + 127) / 128;
  const long tiles = (long)((N + 15) / 16) * n_kt;
  const long blocks = (tiles + 3) / 4;
  if (blocks > 0x7fffffffL) return NS_ERR_BAD_ARG;
  untile_kernel<<<(unsigned)blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)wt, N, K, KT, kt0, n_kt, out_stride, tiles);
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

// dst[dst_idx[i]] = src[src_idx[i]]: token ids sampled by one step become the input ids of the next without a trip
// to the host.
__global__ void scatter_i32_kernel(int* __restrict__ dst, const int* __restrict__ dst_idx, const int* __restrict__ src,
                                   const int* __restrict__ src_idx, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[dst_idx[i]] = src[src_idx[i]];
}
extern "C" int ns_scatter_i32(int* dst, const int* dst_idx, const int* src, const int* src_idx, int n, hipStream_t stream) {
  if (n <= 0) return NS_OK;
  scatter_i32_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, dst_idx, src, src_idx, n);
  return ns_launch_status();
}
