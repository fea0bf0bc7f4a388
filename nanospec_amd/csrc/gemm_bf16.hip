// bfloat16 matrix products on the matrix cores for few rows (decode and short portions):
//   out[M, N] = x[M, K] . w[N, K]^T,  M <= 64,  32-bit accumulation,  K a multiple of 8.
//
// The work is the streaming of w, read exactly once, from a layout made at load time ("tiled") in which every
// load of a wave is one contiguous kilobyte:
//   wt[row tile rt][k tile kt][i = 0..3][lane = 16 g + r][e = 0..7] = w[16 rt + r][128 kt + 32 g + 8 i + e]
// rows padded to a multiple of 16 and k to a multiple of 128 with zeros.  A workgroup owns one row tile; its waves
// take the k tiles in turn (wave v takes kt = v, v + WAVES, ...), so the workgroup as a whole walks through contiguous
// memory, and each streams its share straight into the A operand of v_mfma_f32_16x16x32_bf16 (lane = row r + 16 g
// holds 8 consecutive k of row r); x is the B operand (lane = token m + 16 g), pieces of x beyond K are zero.  Which k
// sits in which of the instruction's 32 slots is free as long as both operands agree.  Partial sums of the waves meet
// in LDS and are added in wave order, so the result does not depend on timing.
//
// Epilogues: plain store (bfloat16 or 32-bit); silu(gate) * up with a second weight matrix read in the same pass
// (reference: model/llama.py:195); rotation and cache write for the stacked q/k/v matrix.
// (reference for the products themselves: the nn.Linear calls of model/llama.py:175,184,195,286)
#include "common.h"
#include "rope.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

#define EPI_STORE 0
#define EPI_SILU_MUL 1
#define EPI_ROPE_KV 2
#define EPI_RESID_NORM 3
#define EPI_GATED_HALF 4
// EPI_GATED_HALF is EPI_SILU_MUL with half the work per workgroup: the 16 rows of a workgroup's matrix instruction are 8
// rows of the gate matrix and the same 8 rows of the up matrix (a lane is free to take its 16 bytes from any row of
// either tiled matrix), placed so that a gate row's sum and its up row's sum come out in the same lane.  Twice as many
// workgroups, each streaming half as much: a compute unit streams at a fixed rate, so a product takes as long as the
// compute unit with the most workgroups, and 14,336 rows are 3.5 workgroups per compute unit of the one kind (as slow as 4)
// and 7 of the other.

// (RopeKvParams, what the q/k/v epilogue needs, and the epilogue's work for one pair of sums: rope.h)

// How a product can take over the work of the norm kernels around it (reference for the norm: model/llama.py:86-95, for
// the sums it sits between: model/llama.py:198-208).  RMS norm is y = w * (r / rms(r)); the division is a factor per
// row, so it can be applied after the product, and the sum of squares of a row can be gathered from the workgroups of
// the product that made r.
//   as producer (EPI_RESID_NORM): r = resid + out (both rounded to bfloat16 as the separate kernels would round them)
//     is stored back into resid, x_next = r * w_next is stored for the next product, and the sum of r^2 over this
//     workgroup's 16 columns goes to ssq_out[row][workgroup].
//   as consumer (ssq_in != null): x is such an x_next; the sums are multiplied by
//     rinv[row] = rsqrt(sum_p ssq_in[row][p] / dim + eps) before the epilogue.
struct NormLink {
  const float* ssq_in;  // [M][parts_in]
  int parts_in;
  float inv_dim, eps;
  bf16_t* resid;        // [M, resid_stride], read and written at this workgroup's columns only
  const bf16_t* w_next; // [N]
  bf16_t* x_next;       // [M, resid_stride]
  float* ssq_out;       // [M][workgroups]
  int resid_stride;
};

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <int MT, int WAVES, int EPI, typename OutT>
__global__ __launch_bounds__(WAVES * 64) void gemm_tiled_kernel(OutT* __restrict__ out, const bf16_t* __restrict__ x,
                                                                 const bf16_t* __restrict__ wt,
                                                                 const bf16_t* __restrict__ wt2, int M, int N, int K,
                                                                 int x_stride, int out_stride, RopeKvParams rk, NormLink nl) {
  constexpr int NACC = EPI == EPI_SILU_MUL ? 2 : 1;
  __shared__ float red[WAVES][NACC * MT][256];
  __shared__ float rinv_s[MT * 16];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // the same in a wave's lanes
  const int r = lane & 15, g = lane >> 4;
  const int tile = EPI == EPI_GATED_HALF ? blockIdx.x >> 1 : blockIdx.x;  // the stored row tile(s) this workgroup reads
  const int n0 = tile * 16;
  const int KT = (K + 127) / 128;
  // What the epilogue needs besides the sums is asked for now and used after the weights have streamed.
  // Consumer: wave v takes rows v, v + WAVES, ...; its lanes take the producer's workgroups in turn.
  constexpr int RPW = (16 + WAVES - 1) / WAVES, PRE = 4;
  // The loads are unconditional, from indices kept inside the arrays, and what lies outside is dropped where the values
  // are used: a load under a condition would be waited for on the spot, before the weights' loads have even started.
  float ssq_pre[RPW][PRE];
  if (nl.ssq_in) {
#pragma unroll
    for (int rr = 0; rr < RPW; ++rr)
#pragma unroll
      for (int i = 0; i < PRE; ++i) {
        const int m = min(wave + rr * WAVES, M - 1), p = min(lane + 64 * i, nl.parts_in - 1);
        ssq_pre[rr][i] = nl.ssq_in[(size_t)m * nl.parts_in + p];
      }
  }
  // Producer: thread e <-> (column n0 + e / 16, row e % 16), one or two elements per thread.
  constexpr int EPT = (256 + WAVES * 64 - 1) / (WAVES * 64);
  float resid_pre[EPT], wnext_pre[EPT];
  if (EPI == EPI_RESID_NORM) {
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int e = min(threadIdx.x + i * WAVES * 64, 255);
      const int n = min(n0 + (e >> 4), N - 1), m = min(e & 15, M - 1);
      resid_pre[i] = (float)nl.resid[(size_t)m * nl.resid_stride + n];
      wnext_pre[i] = (float)nl.w_next[n];
    }
  }
  // EPI_GATED_HALF: rows 4 q + {0, 1} of the instruction are gate rows 8 h + 2 q + {0, 1} of the tile, rows 4 q + {2, 3} the
  // same rows of the up matrix (h = which half of the tile); the sums of row 4 q + j come out in lane group q, element j.
  const int src_row = EPI == EPI_GATED_HALF ? 8 * (blockIdx.x & 1) + 2 * (r >> 2) + (r & 1) : r;
  const bf16_t* wsrc = (EPI == EPI_GATED_HALF && (r & 2)) ? wt2 : wt;
  const bf16_t* wbase = wsrc + (size_t)tile * KT * 2048 + (16 * g + src_row) * 8;
  const bf16_t* w2base = EPI == EPI_SILU_MUL ? wt2 + (size_t)blockIdx.x * KT * 2048 + lane * 8 : nullptr;
  const bf16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xrow[mt] = x + (size_t)min(mt * 16 + r, M - 1) * x_stride + g * 32;

  f32x4 acc[NACC][MT];
#pragma unroll
  for (int a = 0; a < NACC; ++a)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[a][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  struct Stage {
    bf16x8 wf[NACC][4], xf[MT][4];
  };
  auto load = [&](Stage& st, int kt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      st.wf[0][i] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wbase + (size_t)kt * 2048 + i * 512));
      if (EPI == EPI_SILU_MUL) st.wf[NACC - 1][i] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w2base + (size_t)kt * 2048 + i * 512));
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) st.xf[mt][i] = load8(xrow[mt] + kt * 128 + i * 8);
    }
  };
  auto mma = [&](const Stage& st) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int a = 0; a < NACC; ++a)
          acc[a][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(st.wf[a][i], st.xf[mt][i], acc[a][mt], 0, 0, 0);
  };

  const int kt_full = K / 128;  // k tiles that x covers wholly
  Stage s0, s1;
  int kt = wave;
  if (kt < kt_full) load(s0, kt);
  while (kt + WAVES < kt_full) {
    load(s1, kt + WAVES);
    mma(s0);
    if (kt + 2 * WAVES < kt_full) load(s0, kt + 2 * WAVES);
    mma(s1);
    kt += 2 * WAVES;
  }
  if (kt < kt_full) {
    mma(s0);
    kt += WAVES;
  }
  if (kt == kt_full && kt_full < KT) {  // the ragged end of K belongs to exactly one wave
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = kt * 128 + g * 32 + i * 8 < K;
      s0.wf[0][i] = load8(wbase + (size_t)kt * 2048 + i * 512);
      if (EPI == EPI_SILU_MUL) s0.wf[NACC - 1][i] = load8(w2base + (size_t)kt * 2048 + i * 512);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) s0.xf[mt][i] = ok ? load8(xrow[mt] + kt * 128 + i * 8) : zero;
    }
    mma(s0);
  }

#pragma unroll
  for (int a = 0; a < NACC; ++a)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 4; ++j) red[wave][a * MT + mt][lane * 4 + j] = acc[a][mt][j];
  if (nl.ssq_in) {
#pragma unroll
    for (int rr = 0; rr < RPW; ++rr) {
      const int m = wave + rr * WAVES;
      float v = 0.f;
#pragma unroll
      for (int i = 0; i < PRE; ++i) {
        asm volatile("" : "+v"(ssq_pre[rr][i]));  // first used here, after the loop: no arithmetic on it may move up to its load
        v += (m < M && lane + 64 * i < nl.parts_in) ? ssq_pre[rr][i] : 0.f;
      }
      if (m < M)
        for (int p = lane + 64 * PRE; p < nl.parts_in; p += 64) v += nl.ssq_in[(size_t)m * nl.parts_in + p];
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
      if (lane == 0 && m < M) rinv_s[m] = rsqrtf(v * nl.inv_dim + nl.eps);
    }
  }
  __syncthreads();
  if (EPI == EPI_ROPE_KV) {
    // thread e <-> (token m, pair p): the sums of local rows p and p + 8
    const int tiles_per_head = rk.hd / 16;
    const int gh = blockIdx.x / tiles_per_head, jt = blockIdx.x % tiles_per_head;  // head among [q heads | k heads | v heads]
    for (int e = threadIdx.x; e < M * 8; e += WAVES * 64) {
      const int m = e >> 3, p = e & 7;
      const int mt = m >> 4, mr = m & 15;
      // local row r sits at lane (r / 4) * 16 + token, element r % 4
      const int i1 = ((p >> 2) * 16 + mr) * 4 + (p & 3), i2 = (((p + 8) >> 2) * 16 + mr) * 4 + (p & 3);
      float x1 = 0.f, x2 = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) {
        x1 += red[wv][mt][i1];
        x2 += red[wv][mt][i2];
      }
      if (nl.ssq_in) {
        x1 *= rinv_s[m];
        x2 *= rinv_s[m];
      }
      rope_kv_store_pair(rk, out, out_stride, m, gh, jt, p, x1, x2);
    }
    return;
  }
  if (EPI == EPI_RESID_NORM) {
    // thread e <-> (column n0 + e / 16, row e % 16); squares meet in LDS and each row's 16 are added in column order
    __shared__ float sq[16][17];
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const int e = threadIdx.x + i * WAVES * 64;
      if (e >= 256) break;
      const int nl_ = e >> 4, m = e & 15;                 // local column, row
      const int le = (((nl_ >> 2) * 16 + m) << 2) + (nl_ & 3);  // where the product's sums for (row, column) sit
      const int n = n0 + nl_;
      float q = 0.f;
      asm volatile("" : "+v"(resid_pre[i]), "+v"(wnext_pre[i]));  // first used here (see the sums of squares above)
      if (n < N && m < M) {
        float s = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) s += red[wv][0][le];
        const size_t at = (size_t)m * nl.resid_stride + n;
        const bf16_t r = (bf16_t)(resid_pre[i] + (float)(bf16_t)s);
        nl.resid[at] = r;
        nl.x_next[at] = (bf16_t)((float)r * wnext_pre[i]);
        q = (float)r * (float)r;
      }
      sq[m][nl_] = q;
    }
    __syncthreads();
    if (threadIdx.x < M) {
      float v = 0.f;
#pragma unroll
      for (int c = 0; c < 16; ++c) v += sq[threadIdx.x][c];
      nl.ssq_out[(size_t)threadIdx.x * gridDim.x + blockIdx.x] = v;
    }
    return;
  }
  if (EPI == EPI_GATED_HALF) {
    for (int e = threadIdx.x; e < MT * 128; e += WAVES * 64) {
      const int mt = e >> 7, l = (e & 127) >> 1, j = e & 1;  // lane l of the sums holds gate at j, up at 2 + j
      const int n = n0 + 8 * (blockIdx.x & 1) + 2 * (l >> 4) + j, m = mt * 16 + (l & 15);
      if (n >= N || m >= M) continue;
      float s = 0.f, u = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) {
        s += red[wv][mt][l * 4 + j];
        u += red[wv][mt][l * 4 + 2 + j];
      }
      if (nl.ssq_in) {
        s *= rinv_s[m];
        u *= rinv_s[m];
      }
      out[(size_t)m * out_stride + n] = (OutT)(s / (1.f + expf(-s)) * u);
    }
    return;
  }
  for (int e = threadIdx.x; e < MT * 256; e += WAVES * 64) {
    const int mt = e >> 8, le = e & 255;
    const int l = le >> 2, j = le & 3;
    const int n = n0 + (l >> 4) * 4 + j, m = mt * 16 + (l & 15);
    if (n >= N || m >= M) continue;
    float s = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) s += red[wv][mt][le];
    if (nl.ssq_in) s *= rinv_s[m];
    if (EPI == EPI_SILU_MUL) {
      float u = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) u += red[wv][MT + mt][le];
      if (nl.ssq_in) u *= rinv_s[m];
      s = s / (1.f + expf(-s)) * u;
    }
    out[(size_t)m * out_stride + n] = (OutT)s;
  }
}

template <int MT, int WAVES>
static int launch_tiled(void* out, const void* x, const void* w, const void* w2, int M, int N, int K, int x_stride,
                        int out_stride, int epi, int out_f32, const RopeKvParams& rk, const NormLink& nl, hipStream_t stream) {
  const int grid = (N + 15) / 16;
  const bf16_t* xb = (const bf16_t*)x;
  const bf16_t* wb = (const bf16_t*)w;
  const bf16_t* w2b = (const bf16_t*)w2;
  if (epi == EPI_SILU_MUL) {
    if (out_f32) return NS_ERR_UNSUPPORTED;
    gemm_tiled_kernel<MT, WAVES, EPI_SILU_MUL, bf16_t><<<grid, WAVES * 64, 0, stream>>>((bf16_t*)out, xb, wb, w2b, M, N, K, x_stride, out_stride, rk, nl);
  } else if (epi == EPI_GATED_HALF) {
    if (out_f32 || MT != 1) return NS_ERR_UNSUPPORTED;
    gemm_tiled_kernel<1, WAVES, EPI_GATED_HALF, bf16_t><<<2 * grid, WAVES * 64, 0, stream>>>((bf16_t*)out, xb, wb, w2b, M, N, K, x_stride, out_stride, rk, nl);
  } else if (epi == EPI_RESID_NORM) {
    if (out_f32 || MT != 1) return NS_ERR_UNSUPPORTED;
    gemm_tiled_kernel<1, WAVES, EPI_RESID_NORM, bf16_t><<<grid, WAVES * 64, 0, stream>>>((bf16_t*)out, xb, wb, nullptr, M, N, K, x_stride, out_stride, rk, nl);
  } else if (epi == EPI_ROPE_KV) {
    if (out_f32 || MT != 1) return NS_ERR_UNSUPPORTED;
    gemm_tiled_kernel<1, WAVES, EPI_ROPE_KV, bf16_t><<<grid, WAVES * 64, 0, stream>>>((bf16_t*)out, xb, wb, nullptr, M, N, K, x_stride, out_stride, rk, nl);
  } else if (out_f32) {
    gemm_tiled_kernel<MT, WAVES, EPI_STORE, float><<<grid, WAVES * 64, 0, stream>>>((float*)out, xb, wb, nullptr, M, N, K, x_stride, out_stride, rk, nl);
  } else {
    gemm_tiled_kernel<MT, WAVES, EPI_STORE, bf16_t><<<grid, WAVES * 64, 0, stream>>>((bf16_t*)out, xb, wb, nullptr, M, N, K, x_stride, out_stride, rk, nl);
  }
  return ns_launch_status();
}

static int tiled_dispatch(void* out, const void* x, const void* wt, const void* wt2, int M, int N, int K, int x_stride,
                          int out_stride, int epi, int out_f32, int waves, const RopeKvParams& rk, const NormLink& nl, hipStream_t stream) {
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || (K & 7) || (x_stride & 7) || x_stride < K) return NS_ERR_BAD_ARG;
  if (epi != EPI_ROPE_KV && epi != EPI_RESID_NORM && out_stride < N) return NS_ERR_BAD_ARG;
  if (nl.ssq_in && (nl.parts_in <= 0 || M > 16)) return NS_ERR_BAD_ARG;
  if ((epi == EPI_SILU_MUL || epi == EPI_GATED_HALF) && !wt2) return NS_ERR_BAD_ARG;
  const int mt = (M + 15) / 16;
#define NS_TILED(MTV)                                                                                               \
  case MTV:                                                                                                         \
    return waves == 8 ? launch_tiled<MTV, 8>(out, x, wt, wt2, M, N, K, x_stride, out_stride, epi, out_f32, rk, nl, stream)  \
         : waves == 2 ? launch_tiled<MTV, 2>(out, x, wt, wt2, M, N, K, x_stride, out_stride, epi, out_f32, rk, nl, stream)  \
                      : launch_tiled<MTV, 4>(out, x, wt, wt2, M, N, K, x_stride, out_stride, epi, out_f32, rk, nl, stream);
  switch (mt) {
    NS_TILED(1)
    NS_TILED(2)
    NS_TILED(3)
    NS_TILED(4)
  }
#undef NS_TILED
  return NS_ERR_BAD_ARG;
}

// wt (and wt2) in the tiled layout described above; N and K are the sizes of the plain matrix.
// ssq_in (may be null): x holds rows that a norm's weight has scaled but its 1/rms has not; see NormLink.
extern "C" int ns_gemm_tiled_bf16(void* out, const void* x, const void* wt, const void* wt2, int M, int N, int K,
                                  int x_stride, int out_stride, int epi, int out_f32, int waves, const float* ssq_in,
                                  int parts_in, int norm_dim, float eps, hipStream_t stream) {
  if (epi != EPI_STORE && epi != EPI_SILU_MUL && epi != EPI_GATED_HALF) return NS_ERR_BAD_ARG;
  RopeKvParams rk = {};
  NormLink nl = {};
  nl.ssq_in = ssq_in; nl.parts_in = parts_in; nl.inv_dim = norm_dim > 0 ? 1.f / (float)norm_dim : 0.f; nl.eps = eps;
  return tiled_dispatch(out, x, wt, wt2, M, N, K, x_stride, out_stride, epi, out_f32, waves, rk, nl, stream);
}

// The product of up to 16 rows whose result is a block's contribution to the residual stream: resid += x . w^T (in place),
// x_next = resid * w_next, ssq_out[M][(N + 15) / 16] = sums of resid^2 over each workgroup's 16 columns.  See NormLink.
extern "C" int ns_gemm_resid_norm_bf16(void* resid, void* x_next, void* ssq_out, const void* w_next, const void* x,
                                       const void* wt, int M, int N, int K, int x_stride, int resid_stride, int waves,
                                       hipStream_t stream) {
  if (M > 16 || !resid || !x_next || !ssq_out || !w_next || resid_stride < N) return NS_ERR_BAD_ARG;
  RopeKvParams rk = {};
  NormLink nl = {};
  nl.resid = (bf16_t*)resid; nl.w_next = (const bf16_t*)w_next; nl.x_next = (bf16_t*)x_next; nl.ssq_out = (float*)ssq_out;
  nl.resid_stride = resid_stride;
  return tiled_dispatch(resid, x, wt, nullptr, M, N, K, x_stride, resid_stride, EPI_RESID_NORM, 0, waves, rk, nl, stream);
}

// The stacked q/k/v product of up to 16 tokens with rotation and cache write fused in.  ``wt`` holds the stacked matrix with
// its rows permuted as RopeKvParams describes; ``q_out`` [M, >= heads * hd] receives the rotated q.
extern "C" int ns_gemm_qkv_rope_bf16(void* q_out, const void* x, const void* wt, int M, int K, int x_stride, int q_stride,
                                     const int* positions, const int* token_req, const int* block_table, int table_stride,
                                     const float* inv_freq, void* k_cache, void* v_cache, int heads, int kv_heads, int hd,
                                     int rot, int interleaved, float factor, int page_size, int write_kv, int waves,
                                     const float* ssq_in, int parts_in, int norm_dim, float eps, hipStream_t stream) {
  if (M > 16 || hd % 16 || rot % 16 || rot > hd || heads <= 0 || kv_heads <= 0 || page_size <= 0 || q_stride < heads * hd)
    return NS_ERR_BAD_ARG;
  RopeKvParams rk;
  rk.positions = positions; rk.token_req = token_req; rk.block_table = block_table; rk.inv_freq = inv_freq;
  rk.k_cache = (bf16_t*)k_cache; rk.v_cache = (bf16_t*)v_cache; rk.table_stride = table_stride; rk.heads = heads;
  rk.kv_heads = kv_heads; rk.hd = hd; rk.rot = rot; rk.page_size = page_size; rk.write_kv = write_kv;
  rk.form = RopeForm{rot, interleaved ? 1 : 0, factor};
  NormLink nl = {};
  nl.ssq_in = ssq_in; nl.parts_in = parts_in; nl.inv_dim = norm_dim > 0 ? 1.f / (float)norm_dim : 0.f; nl.eps = eps;
  const int N = (heads + 2 * kv_heads) * hd;
  return tiled_dispatch(q_out, x, wt, nullptr, M, N, K, x_stride, q_stride, EPI_ROPE_KV, 0, waves, rk, nl, stream);
}
