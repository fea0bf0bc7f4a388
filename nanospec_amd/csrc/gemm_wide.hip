// bfloat16 matrix products on the matrix cores for 17 to 64 rows, for up to 128 rows of one matrix with one row tile per
// wave (decode at large batch, short portions), and for any number of rows in blocks of 128 with two or four row tiles per
// wave (ns_gemm_rows_bf16: the prompts of models that keep the tiled layout only):
//   out[M, N] = x[M, K] . w[N, K]^T,  32-bit accumulation, weights in the tiled layout of gemm_bf16.hip.
//
// With this many rows the traffic of x counts: a workgroup of 4 waves owns 64 rows of w (16 per wave) and all its
// waves walk through the same k tiles, so that a tile of x (up to 128 tokens x 128 k) is fetched once per workgroup, with
// whole-row loads, into LDS and read from there by every wave in the layout the matrix instruction wants.  The weights
// still go from memory straight into registers, each exactly once.  Since 64 rows per workgroup leave too few workgroups
// to fill the GPU, K is cut into `ksplit` ranges over blockIdx.y; each range writes 32-bit partial sums and a second
// kernel adds the ranges in order and applies the epilogue (store as bfloat16 or 32-bit, or silu(gate) * up).  With a
// single range the first kernel applies the epilogue itself and nothing is written twice.
// (reference for the products: the nn.Linear calls of model/llama.py:175,184,195,286)
#include "common.h"
#include "no_alloc.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

// The x tile in LDS: a row holds its sixteen 8-element pieces in the order 4 i + g for piece 4 g + i (the piece that lane
// group g needs in its i-th matrix instruction), and rows are 32 bytes longer than their data.  A 16-byte LDS read is
// served for lanes 0-7 and 16-23 together, i.e. for eight rows at the columns of g and g + 1: this way those sixteen
// pieces lie in sixteen different groups of four banks.
#define WIDE_XPAD 16                 // elements of padding per row of the x tile in LDS
#define WIDE_XROW (128 + WIDE_XPAD)  // elements per row

// An RMS norm before the product whose 1/rms has no kernel of its own (see NormLink in gemm_bf16.hip): x holds the rows
// scaled by the norm's weight, ssq_in[M][parts_in] partial sums of the rows' squares; the sums of the product are
// multiplied by rinv[row] = rsqrt(sum_p ssq_in[row][p] / dim + eps) before the epilogue.  For at most 16 rows, one range.
struct WideNorm {
  const float* ssq_in = nullptr;
  int parts_in = 0;
  float inv_dim = 0.f, eps = 0.f;
};

// partial[(a * ksplit + s) * M * N + m * N + n]: sum over k range s of matrix a (0: w, 1: w2)
// NT: 16-row tiles of w per wave (64 NT rows per workgroup); each fragment of x read from LDS serves all of them.
// direct_out (only with ksplit == 1): the result goes there, as 32-bit if out_f32, else as bfloat16.
// WAVES: waves per workgroup (the x tile is fetched once for all of them).  A product takes as long as the compute unit
// with the most bytes to stream, so the launcher picks the number that deals the row tiles evenly to the compute units.
// HALF (with w2, NACC == 1, one range of K): a wave's 16 rows are 8 rows of w and the same 8 rows of w2, so that the
// unit of work is half a row tile of each and silu(gate) * up pairs lanes 32 apart.
template <int MT, int NACC, int NT, int WAVES = 4, bool HALF = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_wide_kernel(float* __restrict__ partial, const bf16_t* __restrict__ x,
                                                        const bf16_t* __restrict__ wt, const bf16_t* __restrict__ wt2,
                                                        int M, int N, int K, int x_stride, int ksplit,
                                                        void* __restrict__ direct_out, int out_stride, int out_f32,
                                                        int n_groups, int m_blocks, WideNorm nl) {
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16][WIDE_XROW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int KT = (K + 127) / 128;
  const int row_tiles = (N + 15) / 16;
  // n_groups > 0 (many rows): the launch is one row of workgroups, which go round the eight XCDs in launch order; each XCD
  // takes a contiguous share of the (group of weight rows, block of x rows) pairs, blocks of x fastest, so that the few
  // groups of weight rows it works on at a time stay in its own L2 while the blocks of x pass through.
  int bx = blockIdx.x, bz = blockIdx.z;
  if (n_groups > 0) {
    const int total = n_groups * m_blocks, per = (total + 7) / 8;
    const int t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    if (t >= total) return;
    bx = t / m_blocks;
    bz = t - bx * m_blocks;
  }
  static_assert(!HALF || (NACC == 1 && NT == 1), "half tiles: one accumulator set, one tile per wave");
  constexpr int NTHREADS = WAVES * 64;
  const int unit = bx * WAVES + wave;
  const int rt = HALF ? unit >> 1 : unit * NT;  // first of this wave's row tiles
  const int hh = HALF ? unit & 1 : 0;           // which 8 rows of the tile
  const bool has_rows = rt < row_tiles;
  const int split = blockIdx.y;
  const int per = (KT + ksplit - 1) / ksplit;
  const int kt0 = split * per, kt1 = min(KT, kt0 + per);
  // more than MT * 16 rows of x: blockIdx.z takes them MT * 16 at a time (every block of rows reads the weights again)
  const int m_base = bz * (MT * 16);
  const int m_total = M;
  x += (size_t)m_base * x_stride;
  M = min(MT * 16, M - m_base);

  // (a lane's 16 bytes of a k tile's fragment i lie at i * 512 + (16 g + row) * 8 elements of the tile's block)
  const bf16_t* wbase = HALF ? (r < 8 ? wt : wt2) + (size_t)(has_rows ? rt : 0) * KT * 2048 + (g * 16 + 8 * hh + (r & 7)) * 8
                             : wt + (size_t)(has_rows ? rt : 0) * KT * 2048 + lane * 8;
  const bf16_t* w2base = NACC == 2 ? wt2 + (size_t)(has_rows ? rt : 0) * KT * 2048 + lane * 8 : nullptr;

  const size_t tile_step = (size_t)KT * 2048;  // elements between consecutive row tiles
  bool tile_ok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) tile_ok[t] = rt + t < row_tiles;
  f32x4 acc[NACC][NT][MT];
#pragma unroll
  for (int a = 0; a < NACC; ++a)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[a][t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // The x tile of one k tile: MT*16 rows of 128 k = MT*16*16 pieces of 8; the threads take PER pieces each: thread t
  // takes piece t % 16 of rows t / 16 + (NTHREADS / 16) j, so 16 consecutive threads read one row's 256 contiguous bytes.
  static_assert(NTHREADS % 16 == 0, "a thread keeps its piece of a row over the rows it takes");
  constexpr int XROWS = NTHREADS / 16;                    // rows of the tile that the threads take at a time
  constexpr int PER = (MT * 16 + XROWS - 1) / XROWS;      // pieces per thread (the last ones may lie beyond the tile)
  const int xrow0 = tid >> 4, xcol = (tid & 15) * 8;
  const int xslot = (4 * (tid & 3) + ((tid & 15) >> 2)) * 8;  // where piece tid % 16 = 4 g + i of a row goes in LDS
  // A stage holds what one k tile needs from memory: this wave's fragments of w (and w2) and this thread's pieces of x.
  // DEPTH stages are in flight: the loads of k tile t + DEPTH - 1 are issued before the arithmetic of k tile t.
  constexpr int DEPTH = (NACC * NT >= 4 || MT > 6) ? 2 : 3;  // what the registers hold at two waves per SIMD
  struct Stage {
    bf16x8 wf[NACC][NT][4];
    bf16x8 xr[PER];
  };
  Stage st[DEPTH];
  auto fetch = [&](Stage& sg, int kt) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const size_t off = (tile_ok[t] ? t * tile_step : 0) + (size_t)kt * 2048;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        sg.wf[0][t][i] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(wbase + off + i * 512));
        if (NACC == 2) sg.wf[1][t][i] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w2base + off + i * 512));
      }
    }
#pragma unroll
    // No load stands under a condition (the compiler would wait for it on the spot, and with it for every load in
    // flight): rows beyond M repeat row M - 1, whose sums are never stored, and a piece beyond K is read from inside
    // the row and replaced by zeros when it goes into LDS.
    for (int j = 0; j < PER; ++j) {
      const int m = min(xrow0 + XROWS * j, M - 1);
      const int k = min(kt * 128 + xcol, K - 8);
      sg.xr[j] = *reinterpret_cast<const bf16x8*>(x + (size_t)m * x_stride + k);
    }
  };
  auto step = [&](const Stage& sg, int buf, int kt) {
    const bool in_k = kt * 128 + xcol < K;
    // x pieces into LDS, then every wave multiplies its w fragments with the whole tile.  One barrier per k tile: a
    // wave that writes buffer b for tile t + 2 has passed the barrier of tile t + 1, which every wave reaches only
    // after it has finished reading b for tile t.
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (MT * 16 % XROWS == 0 || xrow0 + XROWS * j < MT * 16) *reinterpret_cast<bf16x8*>(&xs[buf][xrow0 + XROWS * j][xslot]) = in_k ? sg.xr[j] : zero;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8 xf = *reinterpret_cast<const bf16x8*>(&xs[buf][mt * 16 + r][(4 * i + g) * 8]);
#pragma unroll
        for (int a = 0; a < NACC; ++a)
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[a][t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sg.wf[a][t][i], xf, acc[a][t][mt], 0, 0, 0);
      }
  };

  // What the epilogue needs of the norm is asked for now and used after the weights have streamed: wave v takes rows v,
  // v + WAVES, ...; its lanes take the parts in turn.  The loads are unconditional, from indices kept inside the array.
  constexpr int RPW = (16 + WAVES - 1) / WAVES, PRE = 4;
  __shared__ float rinv_s[16];
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
#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d)
    if (kt0 + d < kt1) fetch(st[d], kt0 + d);
  // In the body of the first loop every load is unconditional, so the compiler's count of what may stay in flight is
  // exact there; the last tiles (fewer than two rounds of DEPTH) run with the checks.
  int kt = kt0;
  for (; kt + 2 * DEPTH - 2 < kt1; kt += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      fetch(st[(d + DEPTH - 1) % DEPTH], kt + d + DEPTH - 1);
      step(st[d], (kt + d - kt0) & 1, kt + d);
    }
  }
  for (; kt < kt1; kt += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int cur = kt + d;
      if (cur < kt1) {
        if (cur + DEPTH - 1 < kt1) fetch(st[(d + DEPTH - 1) % DEPTH], cur + DEPTH - 1);
        step(st[d], (cur - kt0) & 1, cur);
      }
    }
  }

  if (nl.ssq_in) {  // (the same for every wave of the launch: all of them pass the barrier)
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
      if (lane == 0 && m < M && m < 16) rinv_s[m] = rsqrtf(v * nl.inv_dim + nl.eps);
    }
    __syncthreads();
  }
  if (!has_rows) return;
  // acc[a][t][mt][j] is the sum for w row 16 (rt + t) + 4 g + j and token 16 mt + r
  const float rinv = (nl.ssq_in && r < M) ? rinv_s[r] : 1.f;  // (with a norm there is one tile of rows: token r)
  if (HALF) {  // rows 4 g + j of the instruction's tile: g < 2 row 8 hh + 4 g + j of w, else row 8 hh + 4 (g - 2) + j of w2
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f32x4 up;
#pragma unroll
      for (int j = 0; j < 4; ++j) up[j] = __shfl_down(acc[0][0][mt][j], 32, 64);
      const int m = mt * 16 + r, n = rt * 16 + 8 * hh + 4 * g;
      if (g >= 2 || m >= M) continue;
      bf16_t* dst = (bf16_t*)direct_out + (size_t)(m_base + m) * out_stride + n;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < N) {
          const float gate = acc[0][0][mt][j] * rinv;
          dst[j] = (bf16_t)(gate / (1.f + expf(-gate)) * (up[j] * rinv));
        }
    }
    return;
  }
  if (direct_out) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r, n = (rt + t) * 16 + g * 4;
        if (m >= M || !tile_ok[t]) continue;
        const int mg = m_base + m;
        f32x4 v = acc[0][t][mt];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] *= rinv;
        if (NACC == 2) {
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = v[j] / (1.f + expf(-v[j])) * (acc[NACC - 1][t][mt][j] * rinv);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < N) {
            if (out_f32) ((float*)direct_out)[(size_t)mg * out_stride + n + j] = v[j];
            else ((bf16_t*)direct_out)[(size_t)mg * out_stride + n + j] = (bf16_t)v[j];
          }
      }
    return;
  }
#pragma unroll
  for (int a = 0; a < NACC; ++a)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r, n = (rt + t) * 16 + g * 4;
        if (m >= M || !tile_ok[t]) continue;
        float* dst = partial + ((size_t)(a * ksplit + split) * m_total + m_base + m) * N + n;
        if (n + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<f32x4*>(dst) = acc[a][t][mt];
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (n + j < N) dst[j] = acc[a][t][mt][j];
        }
      }
}

// out[m][n] = epilogue(sum_s partial[s][m][n]); ranges are added in order.
template <typename OutT, int SILU>
__global__ void gemm_wide_reduce_kernel(OutT* __restrict__ out, const float* __restrict__ partial, int M, int N, int out_stride,
                                        int ksplit) {
  const size_t total = (size_t)M * N;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
    float s = 0.f, u = 0.f;
    for (int k = 0; k < ksplit; ++k) {
      s += partial[(size_t)k * total + e];
      if (SILU) u += partial[(size_t)(ksplit + k) * total + e];
    }
    if (SILU) s = s / (1.f + expf(-s)) * u;
    const size_t m = e / N;
    out[m * out_stride + (e - m * N)] = (OutT)s;
  }
}

template <int MT>
static int launch_wide(float* partial, const bf16_t* x, const bf16_t* wt, const bf16_t* wt2, int M, int N, int K, int x_stride,
                       int ksplit, int nt, int waves, int halves, void* direct_out, int out_stride, int out_f32, WideNorm nl, hipStream_t stream) {
  const int row_tiles = (N + 15) / 16;
  if (halves) {  // (checked by the caller: two matrices, one range of K, one tile per wave, 4 or 7 waves)
    const int units = 2 * row_tiles;
    if (waves == 7)
      gemm_wide_kernel<MT, 1, 1, 7, true><<<dim3((units + 6) / 7, 1), 448, 0, stream>>>(partial, x, wt, wt2, M, N, K, x_stride, 1, direct_out, out_stride, out_f32, 0, 0, nl);
    else
      gemm_wide_kernel<MT, 1, 1, 4, true><<<dim3((units + 3) / 4, 1), 256, 0, stream>>>(partial, x, wt, wt2, M, N, K, x_stride, 1, direct_out, out_stride, out_f32, 0, 0, nl);
    return ns_launch_status();
  }
  if (waves == 3) {  // (checked by the caller: one matrix, one tile per wave)
    gemm_wide_kernel<MT, 1, 1, 3, false><<<dim3((row_tiles + 2) / 3, ksplit), 192, 0, stream>>>(partial, x, wt, nullptr, M, N, K, x_stride, ksplit, direct_out, out_stride, out_f32, 0, 0, nl);
    return ns_launch_status();
  }
  dim3 grid((row_tiles + 4 * nt - 1) / (4 * nt), ksplit);
  if (wt2 && nt == 2)
    gemm_wide_kernel<MT, 2, 2><<<grid, 256, 0, stream>>>(partial, x, wt, wt2, M, N, K, x_stride, ksplit, direct_out, out_stride, out_f32, 0, 0, nl);
  else if (wt2)
    gemm_wide_kernel<MT, 2, 1><<<grid, 256, 0, stream>>>(partial, x, wt, wt2, M, N, K, x_stride, ksplit, direct_out, out_stride, out_f32, 0, 0, nl);
  else if (nt == 2)
    gemm_wide_kernel<MT, 1, 2><<<grid, 256, 0, stream>>>(partial, x, wt, nullptr, M, N, K, x_stride, ksplit, direct_out, out_stride, out_f32, 0, 0, nl);
  else
    gemm_wide_kernel<MT, 1, 1><<<grid, 256, 0, stream>>>(partial, x, wt, nullptr, M, N, K, x_stride, ksplit, direct_out, out_stride, out_f32, 0, 0, nl);
  return ns_launch_status();
}

// 65 to 128 rows: one matrix, one row tile per wave (the x tile takes 72 KiB of LDS at 128 rows), or gate and up by half
// tiles, which need one set of sums where whole tiles of both need two.
template <int MT>
static int launch_wide_tall(float* partial, const bf16_t* x, const bf16_t* wt, const bf16_t* wt2, int M, int N, int K, int x_stride,
                            int ksplit, int waves, int halves, void* direct_out, int out_stride, int out_f32, hipStream_t stream) {
  const WideNorm nl;
  const int row_tiles = (N + 15) / 16;
  if (halves) {  // (checked by the caller: two matrices, one range of K, 4 or 7 waves)
    const int units = 2 * row_tiles;
    if (waves == 7)
      gemm_wide_kernel<MT, 1, 1, 7, true><<<dim3((units + 6) / 7, 1), 448, 0, stream>>>(partial, x, wt, wt2, M, N, K, x_stride, 1, direct_out, out_stride, out_f32, 0, 0, nl);
    else
      gemm_wide_kernel<MT, 1, 1, 4, true><<<dim3((units + 3) / 4, 1), 256, 0, stream>>>(partial, x, wt, wt2, M, N, K, x_stride, 1, direct_out, out_stride, out_f32, 0, 0, nl);
    return ns_launch_status();
  }
  dim3 grid((row_tiles + 3) / 4, ksplit);
  gemm_wide_kernel<MT, 1, 1><<<grid, 256, 0, stream>>>(partial, x, wt, nullptr, M, N, K, x_stride, ksplit, direct_out, out_stride, out_f32, 0, 0, nl);
  return ns_launch_status();
}

// workspace: (wt2 ? 2 : 1) * ksplit * M * N floats (unused with ksplit == 1).  epi 0: store; 1: silu(x.w^T) * (x.w2^T).
// defer (with ksplit > 1 and epi 0): the ranges stay in the workspace as [ksplit][M][N] and nothing is written to out; they
// are added later by ns_wide_reduce or by a norm that reads them (ns_rmsnorm_partial).
// waves: waves per workgroup, 4, or 3 (one matrix, nt 1, up to 64 rows), or 7 (with halves).  halves: gate and up by half row
// tiles (epi 1, one range of K, nt 1, 4 or 7 waves; also for 65 to 128 rows).
static int wide_product(void* out, void* workspace, const void* x, const void* wt, const void* wt2, int M, int N, int K,
                        int x_stride, int out_stride, int epi, int out_f32, int ksplit, int nt, int defer, int waves, int halves,
                        WideNorm nl, hipStream_t stream) {
  if (nl.ssq_in && (M > 16 || ksplit != 1 || nl.parts_in <= 0)) return NS_ERR_BAD_ARG;
  if (halves ? (epi != 1 || ksplit != 1 || nt != 1 || (waves != 4 && waves != 7))
             : (waves != 4 && !(waves == 3 && epi == 0 && nt == 1 && M <= 64)))
    return NS_ERR_BAD_ARG;
  if (M <= 0 || M > 128 || N <= 0 || K <= 0 || (K & 7) || (x_stride & 7) || x_stride < K || out_stride < N) return NS_ERR_BAD_ARG;
  if (M > 64 && ((wt2 != nullptr && !halves) || nt != 1)) return NS_ERR_BAD_ARG;  // 65 to 128 rows: one row tile per wave; two matrices by half tiles only
  if ((epi == 1) != (wt2 != nullptr) || (epi != 0 && epi != 1) || (epi == 1 && out_f32)) return NS_ERR_BAD_ARG;
  const int KT = (K + 127) / 128;
  if (ksplit < 1 || ksplit > KT || ksplit > 65535 || (nt != 1 && nt != 2) || (ksplit > 1 && !workspace)) return NS_ERR_BAD_ARG;
  const int mt = (M + 15) / 16;
  float* part = (float*)workspace;
  void* direct = ksplit == 1 ? out : nullptr;
  int st;
  switch (mt) {
    case 1: st = launch_wide<1>(part, (const bf16_t*)x, (const bf16_t*)wt, (const bf16_t*)wt2, M, N, K, x_stride, ksplit, nt, waves, halves, direct, out_stride, out_f32, nl, stream); break;
    case 2: st = launch_wide<2>(part, (const bf16_t*)x, (const bf16_t*)wt, (const bf16_t*)wt2, M, N, K, x_stride, ksplit, nt, waves, halves, direct, out_stride, out_f32, nl, stream); break;
    case 3: st = launch_wide<3>(part, (const bf16_t*)x, (const bf16_t*)wt, (const bf16_t*)wt2, M, N, K, x_stride, ksplit, nt, waves, halves, direct, out_stride, out_f32, nl, stream); break;
    case 4: st = launch_wide<4>(part, (const bf16_t*)x, (const bf16_t*)wt, (const bf16_t*)wt2, M, N, K, x_stride, ksplit, nt, waves, halves, direct, out_stride, out_f32, nl, stream); break;
    case 5: st = launch_wide_tall<5>(part, (const bf16_t*)x, (const bf16_t*)wt, (const bf16_t*)wt2, M, N, K, x_stride, ksplit, waves, halves, direct, out_stride, out_f32, stream); break;
    case 6: st = launch_wide_tall<6>(part, (const bf16_t*)x, (const bf16_t*)wt, (const bf16_t*)wt2, M, N, K, x_stride, ksplit, waves, halves, direct, out_stride, out_f32, stream); break;
    case 7: st = launch_wide_tall<7>(part, (const bf16_t*)x, (const bf16_t*)wt, (const bf16_t*)wt2, M, N, K, x_stride, ksplit, waves, halves, direct, out_stride, out_f32, stream); break;
    default: st = launch_wide_tall<8>(part, (const bf16_t*)x, (const bf16_t*)wt, (const bf16_t*)wt2, M, N, K, x_stride, ksplit, waves, halves, direct, out_stride, out_f32, stream); break;
  }
  if (st != NS_OK || direct) return st;
  if (defer) return epi == 0 ? NS_OK : NS_ERR_BAD_ARG;
  const size_t total = (size_t)M * N;
  const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
  if (epi == 1)
    gemm_wide_reduce_kernel<bf16_t, 1><<<blocks, 256, 0, stream>>>((bf16_t*)out, part, M, N, out_stride, ksplit);
  else if (out_f32)
    gemm_wide_reduce_kernel<float, 0><<<blocks, 256, 0, stream>>>((float*)out, part, M, N, out_stride, ksplit);
  else
    gemm_wide_reduce_kernel<bf16_t, 0><<<blocks, 256, 0, stream>>>((bf16_t*)out, part, M, N, out_stride, ksplit);
  return ns_launch_status();
}

extern "C" int ns_gemm_wide_bf16(void* out, void* workspace, const void* x, const void* wt, const void* wt2, int M, int N,
                                 int K, int x_stride, int out_stride, int epi, int out_f32, int ksplit, int nt, int defer,
                                 hipStream_t stream) {
  return wide_product(out, workspace, x, wt, wt2, M, N, K, x_stride, out_stride, epi, out_f32, ksplit, nt, defer, 4, 0, WideNorm{}, stream);
}

// The same with the number of waves per workgroup and the unit of work chosen by the caller (see wide_product), so that
// the row tiles can be dealt evenly to the compute units, and with the partial sums of a norm before the product (ssq_in may
// be null; see WideNorm).  halves: up to 128 rows.
extern "C" int ns_gemm_wide_dealt_bf16(void* out, void* workspace, const void* x, const void* wt, const void* wt2, int M, int N,
                                       int K, int x_stride, int out_stride, int epi, int out_f32, int ksplit, int nt, int defer,
                                       int waves, int halves, const float* ssq_in, int parts_in, int norm_dim, float eps,
                                       hipStream_t stream) {
  WideNorm nl;
  nl.ssq_in = ssq_in; nl.parts_in = parts_in; nl.inv_dim = norm_dim > 0 ? 1.f / (float)norm_dim : 0.f; nl.eps = eps;
  return wide_product(out, workspace, x, wt, wt2, M, N, K, x_stride, out_stride, epi, out_f32, ksplit, nt, defer, waves, halves, nl, stream);
}

// ------------------------------------------------------------------ the same product without a workspace argument
// The partial sums of the ranges lie in an array of the library's own (see no_alloc.h).  In host code the array's name is
// only a handle for hipGetSymbolAddress: every GPU has its own copy at its own address, which is looked up once per GPU,
// with that GPU current, and kept; only that address is ever given to a kernel.
static __device__ __align__(256) float scratch[NS_STATIC_SCRATCH_FLOATS];

#define NS_MAX_GPUS 64
static float* scratch_ptr[NS_MAX_GPUS];  // per GPU: the address of its copy of `scratch`, nullptr until looked up

// -> this GPU's copy of the array, or nullptr with *err set.
static float* static_scratch(int* err) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { *err = (int)e; return nullptr; }
  if (dev < 0 || dev >= NS_MAX_GPUS) { *err = NS_ERR_BAD_ARG; return nullptr; }
  float* p = __atomic_load_n(&scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (p) return p;
  void* found = nullptr;
  e = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !found) { *err = e != hipSuccess ? (int)e : NS_ERR_UNSUPPORTED; return nullptr; }
  __atomic_store_n(&scratch_ptr[dev], (float*)found, __ATOMIC_RELEASE);  // two threads at once find the same address
  return (float*)found;
}

extern "C" int ns_static_scratch_init(void) {
  int err = NS_OK;
  return static_scratch(&err) ? NS_OK : err;
}

extern "C" int ns_gemm_wide_bf16_static(void* out, const void* x, const void* wt, const void* wt2, int M, int N, int K,
                                        int x_stride, int out_stride, int epi, int out_f32, int ksplit, int nt,
                                        hipStream_t stream) {
  if (M <= 0 || N <= 0 || ksplit < 1 || !out) return NS_ERR_BAD_ARG;
  float* ws = nullptr;
  if (ksplit > 1) {
    const unsigned long long need = (unsigned long long)(wt2 ? 2 : 1) * (unsigned long long)ksplit * (unsigned long long)M * (unsigned long long)N;
    if (need > NS_STATIC_SCRATCH_FLOATS) return NS_ERR_SCRATCH_TOO_SMALL;
    int err = NS_OK;
    ws = static_scratch(&err);
    if (!ws) return err;
  }
  return wide_product(out, ws, x, wt, wt2, M, N, K, x_stride, out_stride, epi, out_f32, ksplit, nt, 0, 4, 0, WideNorm{}, stream);
}

// Any number of rows, 128 at a time over blockIdx.z, with `nt` row tiles of w per wave (2 or 4; 1 or 2 with wt2): each
// fragment of x read from LDS then serves nt (2 nt with wt2) matrix instructions, which is what many rows need.  Every
// block of 128 rows reads the weights again (from the caches, if the matrix fits them).  For models whose weights are
// kept in the tiled layout only.  Arguments as ns_gemm_wide_bf16.
extern "C" int ns_gemm_rows_bf16(void* out, void* workspace, const void* x, const void* wt, const void* wt2, int M, int N,
                                 int K, int x_stride, int out_stride, int epi, int out_f32, int ksplit, int nt, int defer,
                                 hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || (K & 7) || (x_stride & 7) || x_stride < K || out_stride < N) return NS_ERR_BAD_ARG;
  if ((epi == 1) != (wt2 != nullptr) || (epi != 0 && epi != 1) || (epi == 1 && out_f32)) return NS_ERR_BAD_ARG;
  const int KT = (K + 127) / 128;
  if (ksplit < 1 || ksplit > KT || ksplit > 65535 || (ksplit > 1 && !workspace)) return NS_ERR_BAD_ARG;
  if (wt2 ? (nt != 1 && nt != 2) : (nt != 2 && nt != 4)) return NS_ERR_BAD_ARG;
  const int m_blocks = (M + 127) / 128;
  if (m_blocks > 65535) return NS_ERR_BAD_ARG;
  const int row_tiles = (N + 15) / 16;
  const int n_groups = (row_tiles + 4 * nt - 1) / (4 * nt);
  dim3 grid(8 * ((n_groups * m_blocks + 7) / 8), ksplit, 1);
  float* part = (float*)workspace;
  void* direct = ksplit == 1 ? out : nullptr;
  const bf16_t *xp = (const bf16_t*)x, *w1 = (const bf16_t*)wt, *w2 = (const bf16_t*)wt2;
  if (wt2 && nt == 2)
    gemm_wide_kernel<8, 2, 2><<<grid, 256, 0, stream>>>(part, xp, w1, w2, M, N, K, x_stride, ksplit, direct, out_stride, out_f32, n_groups, m_blocks, WideNorm{});
  else if (wt2)
    gemm_wide_kernel<8, 2, 1><<<grid, 256, 0, stream>>>(part, xp, w1, w2, M, N, K, x_stride, ksplit, direct, out_stride, out_f32, n_groups, m_blocks, WideNorm{});
  else if (nt == 4)
    gemm_wide_kernel<8, 1, 4><<<grid, 256, 0, stream>>>(part, xp, w1, nullptr, M, N, K, x_stride, ksplit, direct, out_stride, out_f32, n_groups, m_blocks, WideNorm{});
  else
    gemm_wide_kernel<8, 1, 2><<<grid, 256, 0, stream>>>(part, xp, w1, nullptr, M, N, K, x_stride, ksplit, direct, out_stride, out_f32, n_groups, m_blocks, WideNorm{});
  int st = ns_launch_status();
  if (st != NS_OK || direct) return st;
  if (defer) return epi == 0 ? NS_OK : NS_ERR_BAD_ARG;
  const size_t total = (size_t)M * N;
  const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
  if (epi == 1)
    gemm_wide_reduce_kernel<bf16_t, 1><<<blocks, 256, 0, stream>>>((bf16_t*)out, part, M, N, out_stride, ksplit);
  else if (out_f32)
    gemm_wide_reduce_kernel<float, 0><<<blocks, 256, 0, stream>>>((float*)out, part, M, N, out_stride, ksplit);
  else
    gemm_wide_reduce_kernel<bf16_t, 0><<<blocks, 256, 0, stream>>>((bf16_t*)out, part, M, N, out_stride, ksplit);
  return ns_launch_status();
}

// out[m][n] = sum over the ranges of partial[s][m][n], added in order.
extern "C" int ns_wide_reduce(void* out, const void* partial, int M, int N, int out_stride, int ksplit, int out_f32,
                              hipStream_t stream) {
  if (M <= 0 || N <= 0 || ksplit < 1 || out_stride < N || !out || !partial) return NS_ERR_BAD_ARG;
  const size_t total = (size_t)M * N;
  const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
  if (out_f32)
    gemm_wide_reduce_kernel<float, 0><<<blocks, 256, 0, stream>>>((float*)out, (const float*)partial, M, N, out_stride, ksplit);
  else
    gemm_wide_reduce_kernel<bf16_t, 0><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const float*)partial, M, N, out_stride, ksplit);
  return ns_launch_status();
}
