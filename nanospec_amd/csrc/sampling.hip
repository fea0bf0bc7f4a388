// From 32-bit logits to a token per row: arg-max for temperature 0, otherwise a draw from the
// soft-max of logits / temperature, optionally restricted to the top-k tokens and to the nucleus
// top-p, by inversion of the cumulative distribution in vocabulary order with a uniform number
// that the host supplies per row.
//
// Reference: engine/engine.py:385-402 (arg-max of the raw logits when the temperature is 0; the
// raw log-probability z[tok] - logsumexp(z); the log-probability under the processed distribution,
// 0 for greedy rows), spec/sampling.py:24-35 (divide by the temperature; a token stays if the
// probability mass of the tokens ranked before it is <= top_p and its rank is < top_k; log-soft-max
// of what stays), spec/sampling.py:38-42 (first index whose cumulative sum exceeds u * total).
//
// The reference ranks by a full sort.  Here the kept set is {i : s_i >= v*} with v* found by
// bisection over the bit patterns of floats: keep(v) = (#{s_j > v} < k) and (mass{s_j > v} <= top_p)
// is monotone in v.  The two agree except that tokens with exactly equal logits at the border are
// kept or dropped together here.
#include "common.h"

#define SP_THREADS 1024

// Order-preserving map between floats and unsigned integers.
__device__ __forceinline__ uint32_t f2ord(float f) {
  uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ord2f(uint32_t o) {
  uint32_t u = (o & 0x80000000u) ? (o & 0x7fffffffu) : ~o;
  return __uint_as_float(u);
}

__global__ __launch_bounds__(SP_THREADS) void sample_kernel(int* __restrict__ out_tok, float* __restrict__ out_logprob,
                                                            float* __restrict__ out_sample_logprob,
                                                            const float* __restrict__ logits, int row_stride,
                                                            const float* __restrict__ temperature,
                                                            const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                            const float* __restrict__ uniform, int vocab) {
  __shared__ float scratch[16];
  __shared__ float prefix[SP_THREADS];
  __shared__ int s_idx;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (size_t)r * row_stride;

  // arg-max of the raw logits (lowest index among equals) and their log-sum-exp, in one pass: every thread keeps the
  // sum of exp(z - its own maximum so far)
  float best = -INFINITY, se = 0.f;
  int best_i = 0x7fffffff;
  auto take = [&](float v, int i) {
    if (v > best) {
      se = se * expf(best - v) + 1.f;  // best = -inf: se is still 0
      best = v;
      best_i = i;
    } else if (v > -INFINITY) {
      se += expf(v - best);
    }
  };
  if ((((uintptr_t)z) & 15) == 0) {
    const int n4 = vocab >> 2;
    const float4* z4 = reinterpret_cast<const float4*>(z);
    for (int i = tid; i < n4; i += SP_THREADS) {
      const float4 v = z4[i];
      take(v.x, 4 * i);
      take(v.y, 4 * i + 1);
      take(v.z, 4 * i + 2);
      take(v.w, 4 * i + 3);
    }
    for (int i = 4 * n4 + tid; i < vocab; i += SP_THREADS) take(z[i], i);
  } else {
    for (int i = tid; i < vocab; i += SP_THREADS) take(z[i], i);
  }
  const float zmax = block_max(best, scratch);
  if (tid == 0) s_idx = 0x7fffffff;
  __syncthreads();
  if (best == zmax) atomicMin(&s_idx, best_i);
  const float lse = zmax + logf(block_sum(best > -INFINITY ? se * expf(best - zmax) : 0.f, scratch));  // barriers inside publish s_idx
  const int amax = s_idx < vocab ? s_idx : 0;  // a row without a single comparable value (all NaN or -inf) names token 0
  const float T = temperature[r];
  if (T <= 0.f) {
    if (tid == 0) {
      out_tok[r] = amax;
      out_logprob[r] = z[amax] - lse;
      out_sample_logprob[r] = 0.f;
    }
    return;
  }

  const float smax = zmax / T;
  const int k = top_k ? top_k[r] : 0;
  const float pp = top_p ? top_p[r] : 1.f;
  float cut = -INFINITY;  // tokens with s >= cut stay
  if (k > 0 || pp < 1.f) {
    float tot = 0.f;
    for (int i = tid; i < vocab; i += SP_THREADS) tot += expf(z[i] / T - smax);
    tot = block_sum(tot, scratch);
    // smallest ordered key x with keep(ord2f(x)); keep(max) holds (nothing is above the maximum)
    uint32_t lo = 0u, hi = f2ord(smax);
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      const float v = ord2f(mid);
      float cnt = 0.f, mass = 0.f;
      for (int i = tid; i < vocab; i += SP_THREADS) {
        const float s = z[i] / T;
        if (s > v) { cnt += 1.f; mass += expf(s - smax); }
      }
      cnt = block_sum(cnt, scratch);
      mass = block_sum(mass, scratch);
      const bool keep = (k <= 0 || cnt < (float)k) && (mass / tot <= pp);
      if (keep) hi = mid; else lo = mid + 1;
    }
    cut = ord2f(lo);
  }

  // inverse CDF in vocabulary order: each thread owns a contiguous range
  const int per = (vocab + SP_THREADS - 1) / SP_THREADS;
  const int i0 = min(vocab, tid * per), i1 = min(vocab, i0 + per);
  float mine = 0.f;
  int last_kept = -1;
  for (int i = i0; i < i1; ++i) {
    const float s = z[i] / T;
    if (s >= cut) { mine += expf(s - smax); last_kept = i; }
  }
  prefix[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float run = 0.f;
    for (int i = 0; i < SP_THREADS; ++i) { const float v = prefix[i]; prefix[i] = run; run += v; }
    scratch[0] = run;
    s_idx = 0x7fffffff;
  }
  __syncthreads();
  const float total = scratch[0];
  const float target = uniform[r] * total;
  float run = prefix[tid];
  for (int i = i0; i < i1; ++i) {
    const float s = z[i] / T;
    if (s >= cut) {
      run += expf(s - smax);
      if (run > target) { atomicMin(&s_idx, i); break; }
    }
  }
  __syncthreads();
  int tok = s_idx;
  if (tok == 0x7fffffff) {  // u * total rounded up to the total: the last token that stayed
    __syncthreads();
    if (tid == 0) s_idx = -1;
    __syncthreads();
    if (last_kept >= 0) atomicMax(&s_idx, last_kept);
    __syncthreads();
    tok = s_idx;
    if (tok < 0) tok = amax;  // nothing stayed (a row of NaN)
  }
  if (tid == 0) {
    out_tok[r] = tok;
    out_logprob[r] = z[tok] - lse;
    out_sample_logprob[r] = z[tok] / T - smax - logf(total);
  }
}

extern "C" int ns_sample(int* out_tok, float* out_logprob, float* out_sample_logprob, const float* logits, int row_stride,
                         const float* temperature, const int* top_k, const float* top_p, const float* uniform, int rows,
                         int vocab, hipStream_t stream) {
  if (rows <= 0 || vocab <= 0 || row_stride < vocab) return NS_ERR_BAD_ARG;
  sample_kernel<<<rows, SP_THREADS, 0, stream>>>(out_tok, out_logprob, out_sample_logprob, logits, row_stride, temperature,
                                                 top_k, top_p, uniform, vocab);
  return ns_launch_status();
}
