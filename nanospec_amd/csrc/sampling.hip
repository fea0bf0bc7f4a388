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
#define SP_CANDIDATES 8192  // tokens near the maximum that the top-k / top-p search keeps in LDS
#define SP_MARGINS 4        // margins below the maximum that are tried for them, widest first
__device__ __forceinline__ float sp_margin(int d) { return d == 0 ? 16.f : d == 1 ? 8.f : d == 2 ? 4.f : 2.f; }

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
  constexpr int WAVES = SP_THREADS / NS_WAVE;
  __shared__ float scratch[16];
  __shared__ float chunk_sum[WAVES];
  __shared__ int chunk_last[WAVES];
  __shared__ int s_idx;
  __shared__ float cand[SP_CANDIDATES];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (size_t)r * row_stride;
  const bool wide = (((uintptr_t)z) & 15) == 0;
  const int n4 = wide ? vocab >> 2 : 0;
  const float4* z4 = reinterpret_cast<const float4*>(z);

  // First pass: the arg-max of the raw logits, lowest index among equals (a thread meets its indices in rising order).
  // Second pass: the sum of exp(z - max).  Two cheap passes instead of one that rescales a running sum at every element:
  // the row is read by a single compute unit and its arithmetic, not the memory, sets the time.
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  auto take = [&](float v, int i) {
    if (v > best) {
      best = v;
      best_i = i;
    }
  };
  for (int i = tid; i < n4; i += SP_THREADS) {
    const float4 v = z4[i];
    take(v.x, 4 * i);
    take(v.y, 4 * i + 1);
    take(v.z, 4 * i + 2);
    take(v.w, 4 * i + 3);
  }
  for (int i = 4 * n4 + tid; i < vocab; i += SP_THREADS) take(z[i], i);
  const float zmax = block_max(best, scratch);
  if (tid == 0) s_idx = 0x7fffffff;
  __syncthreads();
  if (best == zmax) atomicMin(&s_idx, best_i);
  float se = 0.f;
  auto add = [&](float v) {
    if (v > -INFINITY) se += __expf(v - zmax);  // not for NaN
  };
  for (int i = tid; i < n4; i += SP_THREADS) {
    const float4 v = z4[i];
    add(v.x);
    add(v.y);
    add(v.z);
    add(v.w);
  }
  for (int i = 4 * n4 + tid; i < vocab; i += SP_THREADS) add(z[i]);
  const float lse = zmax + logf(block_sum(zmax > -INFINITY ? se : 0.f, scratch));  // barriers inside publish s_idx
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
    // keep(v) = (#{s_j > v} < k) and (mass{s_j > v} <= top_p * total) is monotone in v; the cut is the smallest v (as an
    // ordered bit pattern) for which it holds.  Each probe of the bisection is a sum over the tokens above v.  Where the cut
    // lies among the few tokens within a margin of the maximum, those are first gathered into LDS (in an order that is
    // the same in every run) and the probes only walk them; otherwise the probes walk the whole row.
    float tot = 0.f;
    float cnt_m[SP_MARGINS], mass_m[SP_MARGINS];
#pragma unroll
    for (int d = 0; d < SP_MARGINS; ++d) cnt_m[d] = mass_m[d] = 0.f;
    for (int i = tid; i < vocab; i += SP_THREADS) {
      const float sv = z[i] / T;
      const float e = expf(sv - smax);
      tot += e;
#pragma unroll
      for (int d = 0; d < SP_MARGINS; ++d)
        if (sv > smax - sp_margin(d)) { cnt_m[d] += 1.f; mass_m[d] += e; }
    }
    tot = block_sum(tot, scratch);
    int use = -1;  // the widest margin whose tokens fit the LDS array
    float cnt_u = 0.f, mass_u = 0.f;
#pragma unroll
    for (int d = 0; d < SP_MARGINS; ++d) {
      const float c = block_sum(cnt_m[d], scratch), m = block_sum(mass_m[d], scratch);
      if (use < 0 && c <= (float)SP_CANDIDATES) { use = d; cnt_u = c; mass_u = m; }
    }
    auto keep = [&](float cnt, float mass) { return (k <= 0 || cnt < (float)k) && (mass / tot <= pp); };
    uint32_t lo = 0u, hi = f2ord(smax);  // keep(max) holds: nothing is above the maximum
    bool gathered = false;
    if (use >= 0) {
      const float tau = smax - sp_margin(use);
      if (keep(cnt_u, mass_u)) {
        hi = f2ord(tau);  // the cut lies at or below the margin: probe the whole row, from there down
      } else {
        lo = f2ord(tau) + 1;  // the cut lies above it, among the gathered tokens
        gathered = true;
      }
    }
    int n_cand = 0;
    if (gathered) {
      // thread t gathers its tokens t, t + 1024, ... in that order behind those of the threads before it
      int mine_n = 0;
      const float tau = smax - sp_margin(use);
      for (int i = tid; i < vocab; i += SP_THREADS) mine_n += (z[i] / T > tau) ? 1 : 0;
      int incl = mine_n;
#pragma unroll
      for (int o = 1; o < NS_WAVE; o <<= 1) {
        const int t = __shfl_up(incl, o, NS_WAVE);
        if ((tid & (NS_WAVE - 1)) >= o) incl += t;
      }
      __syncthreads();
      if ((tid & (NS_WAVE - 1)) == NS_WAVE - 1) chunk_last[tid / NS_WAVE] = incl;
      __syncthreads();
      int at = incl - mine_n;
      for (int j = 0; j < tid / NS_WAVE; ++j) at += chunk_last[j];
      for (int j = 0; j < WAVES; ++j) n_cand += chunk_last[j];
      for (int i = tid; i < vocab; i += SP_THREADS) {
        const float sv = z[i] / T;
        if (sv > tau && at < SP_CANDIDATES) cand[at++] = sv;
      }
      n_cand = min(n_cand, SP_CANDIDATES);
      __syncthreads();
    }
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      const float v = ord2f(mid);
      float cnt = 0.f, mass = 0.f;
      if (gathered) {
        for (int i = tid; i < n_cand; i += SP_THREADS) {
          const float sv = cand[i];
          if (sv > v) { cnt += 1.f; mass += expf(sv - smax); }
        }
      } else {
        for (int i = tid; i < vocab; i += SP_THREADS) {
          const float sv = z[i] / T;
          if (sv > v) { cnt += 1.f; mass += expf(sv - smax); }
        }
      }
      cnt = block_sum(cnt, scratch);
      mass = block_sum(mass, scratch);
      if (keep(cnt, mass)) hi = mid; else lo = mid + 1;
    }
    cut = ord2f(lo);
  }

  // Inverse CDF in vocabulary order.  Every wave owns a contiguous chunk (a multiple of 256 tokens) and adds up what
  // stays of it, its lanes reading neighbouring tokens; then the chunk in which the running sum passes u * total is found.
  const bool filtered = cut > -INFINITY;
  const float inv_t = 1.f / T;
  // what a token weighs and whether it stays; without a cut everything finite stays and the weight needs no division
  auto weigh = [&](float v, bool& kept) -> float {
    if (filtered) {
      const float sv = v / T;  // the very expression whose values the cut was found among
      kept = sv >= cut;
      return kept ? expf(sv - smax) : 0.f;
    }
    kept = v > -INFINITY;  // neither NaN nor a token that was masked out
    return kept ? __expf((v - zmax) * inv_t) : 0.f;
  };
  const int lane = tid & (NS_WAVE - 1), wave = tid / NS_WAVE;
  const int chunk = (((vocab + WAVES - 1) / WAVES) + 4 * NS_WAVE - 1) & ~(4 * NS_WAVE - 1);
  const int c0 = min(vocab, wave * chunk), c1 = min(vocab, c0 + chunk);
  float mine = 0.f;
  int last_kept = -1;
  auto count = [&](float v, int i) {
    bool kept;
    mine += weigh(v, kept);
    if (kept) last_kept = i;
  };
  const int c4 = wide ? (c1 - c0) >> 2 : 0;  // 16-byte pieces of the chunk (it starts at a multiple of 256 tokens)
  for (int q = lane; q < c4; q += NS_WAVE) {
    const float4 v = z4[(c0 >> 2) + q];
    const int i = c0 + 4 * q;
    count(v.x, i);
    count(v.y, i + 1);
    count(v.z, i + 2);
    count(v.w, i + 3);
  }
  for (int i = c0 + 4 * c4 + lane; i < c1; i += NS_WAVE) count(z[i], i);
  mine = wave_sum(mine);
#pragma unroll
  for (int o = NS_WAVE / 2; o > 0; o >>= 1) last_kept = max(last_kept, __shfl_xor(last_kept, o, NS_WAVE));
  if (lane == 0) {
    chunk_sum[wave] = mine;
    chunk_last[wave] = last_kept;
  }
  __syncthreads();
  float total = 0.f;
  for (int j = 0; j < WAVES; ++j) total += chunk_sum[j];
  const float target = uniform[r] * total;
  int sel = -1, last_all = -1;
  float before = 0.f, sel_before = 0.f;
  for (int j = 0; j < WAVES; ++j) {
    if (sel < 0 && before + chunk_sum[j] > target) {
      sel = j;
      sel_before = before;
    }
    before += chunk_sum[j];
    last_all = max(last_all, chunk_last[j]);
  }
  // The chunk in which the passing lies is cut once more, into a piece per wave; the piece in which it lies is walked by
  // its wave alone: the sums of eight runs of 64 tokens at a time (their loads and lane exchanges do not wait for one
  // another), then a scan over the lanes of the run in which the passing lies.
  constexpr int AHEAD = 8;
  const int piece = chunk / WAVES;  // a multiple of 16 tokens
  const int s_lo = sel < 0 ? 0 : min(vocab, sel * chunk), s_hi = sel < 0 ? 0 : min(vocab, s_lo + chunk);
  const int p0 = min(s_hi, s_lo + wave * piece), p1 = min(s_hi, p0 + piece);
  __syncthreads();  // chunk_sum and chunk_last have been read by everyone: they now hold the pieces
  int tok = -1, owner = -1;
  if (sel >= 0) {
    float psum = 0.f;
    int plast = -1;
    for (int b0 = p0; b0 < p1; b0 += AHEAD * NS_WAVE) {
      float v[AHEAD];
#pragma unroll
      for (int j = 0; j < AHEAD; ++j) v[j] = z[min(b0 + j * NS_WAVE + lane, p1 - 1)];  // no load under a condition
#pragma unroll
      for (int j = 0; j < AHEAD; ++j) {
        bool kept;
        const float w = weigh(v[j], kept);
        if (b0 + j * NS_WAVE + lane < p1) {
          psum += w;
          if (kept) plast = b0 + j * NS_WAVE + lane;
        }
      }
    }
    psum = wave_sum(psum);
#pragma unroll
    for (int o = NS_WAVE / 2; o > 0; o >>= 1) plast = max(plast, __shfl_xor(plast, o, NS_WAVE));
    if (lane == 0) {
      chunk_sum[wave] = psum;
      chunk_last[wave] = plast;
    }
  }
  __syncthreads();
  if (sel < 0) {  // u * total rounded up to the total: the last token that stayed
    tok = last_all;
  } else {
    float run = sel_before, run0 = 0.f;
    int last_in_chunk = -1;
    for (int j = 0; j < WAVES; ++j) {
      if (owner < 0 && run + chunk_sum[j] > target) {
        owner = j;
        run0 = run;
      }
      run += chunk_sum[j];
      last_in_chunk = max(last_in_chunk, chunk_last[j]);
    }
    if (owner < 0) {  // the sums of the two passes round differently: the passing lies at the chunk's end
      tok = last_in_chunk;
    } else if (wave == owner) {
      run = run0;
      int last_here = -1;
      for (int b0 = p0; b0 < p1 && tok < 0; b0 += AHEAD * NS_WAVE) {
        float p[AHEAD], sum[AHEAD];
        bool kept[AHEAD];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) p[j] = z[min(b0 + j * NS_WAVE + lane, p1 - 1)];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
          p[j] = weigh(p[j], kept[j]);
          if (b0 + j * NS_WAVE + lane >= p1) {
            kept[j] = false;
            p[j] = 0.f;
          }
        }
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) sum[j] = wave_sum(p[j]);  // eight independent chains of lane exchanges
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
          if (tok >= 0) break;
          const int b = b0 + j * NS_WAVE;
          const unsigned long long stays = __ballot(kept[j]);
          if (run + sum[j] > target) {  // the passing lies in these 64 tokens: inclusive sums over the lanes find it
            float scan = p[j];
#pragma unroll
            for (int o = 1; o < NS_WAVE; o <<= 1) {
              const float t = __shfl_up(scan, o, NS_WAVE);
              if (lane >= o) scan += t;
            }
            const unsigned long long hit = __ballot(kept[j] && run + scan > target);
            // (the scan and the sum round differently: without a hit the passing is the last token here that stayed)
            tok = hit ? b + __ffsll((long long)hit) - 1 : b + 63 - __clzll((long long)stays);
          } else {
            if (stays) last_here = b + 63 - __clzll((long long)stays);
            run += sum[j];
          }
        }
      }
      if (tok < 0) tok = last_here;  // again the rounding: the passing lies at the piece's end
    }
  }
  const bool by_first = sel < 0 || owner < 0;  // every thread knows the token; else only the wave that walked does
  if (by_first ? tid == 0 : (wave == owner && lane == 0)) {
    if (tok < 0) tok = amax;  // nothing stayed (a row of NaN)
    out_tok[r] = tok;
    out_logprob[r] = z[tok] - lse;
    out_sample_logprob[r] = (filtered ? z[tok] / T - smax : (z[tok] - zmax) * inv_t) - logf(total);
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
