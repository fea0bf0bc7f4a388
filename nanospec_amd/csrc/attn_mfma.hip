// Soft-max attention over the paged bfloat16 cache on the matrix cores, for prefill portions and for
// decode, compiled for one head size (NS_HEAD_DIM, a multiple of 16 up to 256) and one page size (NS_PAGE_SIZE).
//
// One wave owns one tile of 16 "columns".  A column is a (query token, query head) pair of one
// request and one key/value head: hp consecutive heads of the group times 16/hp consecutive tokens.
// Prefill portions run with hp = 1 (16 tokens of one head), decode with hp = the group size, so
// that all query heads that share a key/value head share each load of it.
// (reference: model/attention.py:22-43 for what is computed, :86-101 for the two modes)
//
// Everything is kept transposed so that a column is always lane % 16:
//   S^T[key][col] = K[key][:] . Q[col][:]        A = K tile (rows = keys, straight from the page),
//                                                B = Q^T (lane holds 8 channels of its column)
//   soft-max over keys: the 8 keys a lane holds, then across the 4 lane groups (xor 16, 32)
//   O^T[ch][col] += V^T[ch][key] . P^T[key][col]  A = V^T tile, which the cache stores as
//                                                [page][kv head][channel][token]: 4 consecutive
//                                                tokens per 8-byte load; B = P^T is exactly the
//                                                layout S^T came out in.
// The running maximum, the running sum and the output accumulators of a column therefore live in
// the lanes of that column and are rescaled without any exchange.  Keys are walked in blocks of 32;
// the loads of the next block are issued before the arithmetic of the current one.
//
// Query at position p sees keys max(0, p - window + 1) .. p.  Scores, soft-max and sums are 32-bit.
// With splits > 1 the keys of a tile are cut into `splits` contiguous ranges of whole 32-key blocks;
// each range writes its un-normalised output, maximum and sum, and a second small kernel joins them.
//
// Three kernels: attn_mfma_kernel (a wave per tile, or a workgroup per tile for decode rows), attn_prefill_kernel
// (prompt portions in tiles of 32 tokens, four heads of a group share each block of keys through LDS) and, for head
// sizes 64 and 128 and pages of 8 tokens or more, attn_prefill32_kernel in attn_prefill32.h (the same sharing on the
// 32x32 matrix instruction with keys and values loaded straight into LDS).  Compiled with -DNS_PREFILL16 the second
// serves those head sizes too: that is for measurements of one against the other.
#include "common.h"
#include <type_traits>

#if !defined(NS_HEAD_DIM) || !defined(NS_PAGE_SIZE)
#error "compile with -DNS_HEAD_DIM=<multiple of 16> -DNS_PAGE_SIZE=<power of two from 4>"
#endif
constexpr int HD = NS_HEAD_DIM;
constexpr int PS = NS_PAGE_SIZE;  // tokens per cache page: a constant, so that page arithmetic is shifts and offsets are immediates
static_assert(PS >= 4 && (PS & (PS - 1)) == 0, "page size must be a power of two from 4");
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 up to 256");
constexpr int DT = HD / 16;           // 16-channel tiles of the output
constexpr bool WIDE = HD % 32 == 0;   // q.k with the k=32 instruction, else with k=16
constexpr int NQ = WIDE ? HD / 32 : HD / 16;  // q.k instructions per 16-key tile
constexpr int TILE_INTS = 8;          // ints per tile descriptor

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

// A tile descriptor, filled on the host: {request, first token of the tile among the request's tokens of this step
// (tiles of one request follow each other every 16 qt / hp tokens),
// row of the request's first token in the batch, tokens of the request in this step, keys after this step,
// for decode tiles the keys that all decode rows of the step read together over all layers, 0, 0}.
struct AttnParams {
  bf16_t* out;        // [tokens, heads, HD]
  float* part_o;      // [n_tiles * (16 / hp) * heads, splits, HD]   (splits > 1)
  float* part_ml;     // [n_tiles * (16 / hp) * heads, splits, 2]
  const bf16_t* q;    // row t at q + t * q_stride, head h at + h * HD
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  const int* tiles;   // [n_tiles][TILE_INTS]
  const int* block_table;
  int q_stride, table_stride, n_tiles, heads, kv_heads, hp, splits, window;
  int near;          // every byte of the key pool and of the value pool lies within 4 GiB of its start, a page's id and a
                     // page's bytes are below 2^24: byte offsets are then 32-bit and one 24-bit multiply-add each
  float scale_log2;  // softmax scale * log2(e)
};

// 2^x by the hardware instruction alone: arguments here are <= 0, and results below the normal range may flush to 0.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ int wave_max_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}

template <bool NT, typename V>
__device__ __forceinline__ V ld(const V* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}

// The operands of one block of 32 keys as they come from memory.
struct KVBlock {
  bf16x8 kw[WIDE ? 2 * NQ : 1];  // [tile t][i]
  s16x4 kn[WIDE ? 1 : 2 * NQ];
  bf16x4 v[DT][2];               // [channel tile][keys 4g.. of tile 0 | of tile 1]
};

// QT: tiles of 16 columns per wave (2 only with hp == 1: 32 tokens of one head share every load of K and V).
// PREFETCH: the loads of the next key block are issued before the arithmetic of the current one.
// COOP: the four waves of a workgroup share one tile and one key range and take its 32-key blocks in turn; their
// results meet in LDS.  Decode is bound by the latency of a wave's chain of loads, so the chain is made four times
// shorter without more work for the kernel that joins the ranges.
// NT: keys and values are read with non-temporal loads.  A step reads every layer's keys and values once; if all of them
// together fit the memory-side cache they are still there at the next step and plain loads find them, otherwise they only
// push other data out and non-temporal loads are the faster ones (6.1 against 5.7 TB/s at batch 64 and 3,072 keys of the
// 8B shape).  The kernel chooses by the number of keys over all layers, which the host leaves in the tiles.
template <int QT, bool PREFETCH, bool COOP, bool NT>
__device__ __forceinline__ void attn_tiles(const AttnParams& a) {
  // what is the same in all lanes of a wave is said to be so (readfirstlane): branches on it are then scalar ones
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, g = lane >> 4;
  const int G = a.heads / a.kv_heads;
  const int hblks = (G + a.hp - 1) / a.hp;
  const int ny = a.kv_heads * hblks;
  const long item = COOP ? (long)blockIdx.x : (long)blockIdx.x * 4 + wave;
  if (item >= (long)a.n_tiles * a.splits * ny) return;
  const int y = (int)(item % ny);
  const long ts = item / ny;
  // tiles are listed in the order of the tokens; the last ones see the most keys, so they start first
  const int split = (int)(ts % a.splits), tile = a.n_tiles - 1 - (int)(ts / a.splits);
  const int kvh = y / hblks, hblk = y % hblks;
  const int4 info = *reinterpret_cast<const int4*>(a.tiles + (size_t)tile * TILE_INTS);
  const int b = info.x, t0 = info.y, q0 = info.z, n = info.w;
  const int kv_len = a.tiles[(size_t)tile * TILE_INTS + 4];
  const int* table = a.block_table + (size_t)b * a.table_stride;
  constexpr int psh = __builtin_ctz(PS), pmask = PS - 1;

  // this lane's columns: column c of sub-tile u
  const int tt0 = c / a.hp;  // token of the tile (sub-tile 0)
  const int hin = hblk * a.hp + c % a.hp;
  const int head = kvh * G + (hin < G ? hin : 0);
  bool col_ok[QT];
  int pos[QT], lo[QT];
  int whi = 0, wlo = 0x7fffffff, full_hi = 0x7fffffff, full_lo = 0;
#pragma unroll
  for (int u = 0; u < QT; ++u) {
    const int ti = t0 + u * (16 / a.hp) + tt0;
    col_ok[u] = ti < n && hin < G;
    pos[u] = col_ok[u] ? kv_len - n + ti : -1;
    lo[u] = (col_ok[u] && a.window > 0) ? max(0, pos[u] - a.window + 1) : 0;
    whi = max(whi, wave_max_i(pos[u]) + 1);                       // keys [wlo, whi) are seen by some column
    wlo = min(wlo, wave_min_i(col_ok[u] ? lo[u] : 0x7fffffff));
    full_hi = min(full_hi, wave_min_i(col_ok[u] ? pos[u] : 0x7fffffff));  // keys <= full_hi are seen by every column
    full_lo = max(full_lo, wave_max_i(lo[u]));                             // ... if they are >= full_lo
  }

  int kb0 = whi > 0 ? wlo / 32 : 0, kb1 = whi > 0 ? (whi + 31) / 32 : 0;
  if (a.splits > 1) {
    // More than 16 ranges (a launch of few tiles, made for long rows of keys) are only used from 8,192 keys on: below
    // that the ranges beyond the sixteenth stay empty and the others are as long as a launch of 16 would make them.
    const int blocks = kb1 - kb0;
    const int ranges = (a.splits > 16 && blocks < 256) ? 16 : a.splits;
    const int per = (blocks + ranges - 1) / ranges;
    kb0 = kb0 + split * per;
    kb1 = min(kb1, kb0 + per);
  }
  kb0 = __builtin_amdgcn_readfirstlane(kb0);
  kb1 = __builtin_amdgcn_readfirstlane(kb1);

  // Q^T fragments of this lane's columns
  bf16x8 qw[QT][WIDE ? NQ : 1];
  s16x4 qn[QT][WIDE ? 1 : NQ];
#pragma unroll
  for (int u = 0; u < QT; ++u) {
    const int ti = t0 + u * (16 / a.hp) + tt0;
    const bf16_t* qrow = a.q + (size_t)(q0 + (col_ok[u] ? ti : 0)) * a.q_stride + head * HD;
    if (WIDE) {
#pragma unroll
      for (int i = 0; i < NQ; ++i) {
        qw[u][i] = *reinterpret_cast<const bf16x8*>(qrow + i * 32 + g * 8);
        if (!col_ok[u]) qw[u][i] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    } else {
#pragma unroll
      for (int i = 0; i < NQ; ++i) {
        qn[u][i] = *reinterpret_cast<const s16x4*>(qrow + i * 16 + g * 4);
        if (!col_ok[u]) qn[u][i] = s16x4{0, 0, 0, 0};
      }
    }
  }

  f32x4 o[QT][DT];
  float m[QT], lsum[QT];
#pragma unroll
  for (int u = 0; u < QT; ++u) {
    m[u] = -INFINITY;
    lsum[u] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[u][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int qlo = wlo & ~3, qhi = (whi - 1) & ~3;  // first and last 4-key group that holds a seen key
  const size_t kv_row = (size_t)a.kv_heads * HD;   // elements per token of a page
  const bf16_t* kbase = a.k_cache + (((size_t)kvh * HD) << psh) + (WIDE ? g * 8 : g * 4);  // K pages: [page][kv head][token][HD]
  const bf16_t* vbase = a.v_cache + (((size_t)kvh * HD + c) << psh);
  constexpr size_t v_step = (size_t)16 * PS;  // elements between channel tiles of a V page

  // The page ids of up to 64 consecutive pages are held one per lane and handed round by lane exchange, so that the
  // chain of loads of a block is one load long (keys and values) rather than two (block table, then keys and values).
  // The ids of the 64 pages after those are asked for at the same time and taken over when a block reaches them: the
  // lane exchange then never reads a register that a load may still be writing, so nothing waits for the loads in
  // flight (a wait for the page ids would be a wait for all the keys and values asked for before them).
  const int last_page = max(whi - 1, 0) >> psh;
  int page_base = __builtin_amdgcn_readfirstlane((kb0 * 32) >> psh);
  int my_page = table[min(page_base + lane, last_page)];
  int next_pages = table[min(page_base + 64 + lane, last_page)];
  asm volatile("" : "+v"(my_page));  // here, once, the first ids are waited for (on every path into the loops below)
  auto page_of = [&](int key) { return __shfl(my_page, (key >> psh) - page_base, 64); };

  // Issue the loads of block kb: keys, values.  Addresses are kept inside held pages: a key outside [wlo, whi) is masked
  // anyway.
  // A wave's blocks come in rising order, the first one's first page is page_base, and a block's pages never straddle
  // a multiple of 64 pages from there (32 keys are a power of two of pages, or a part of one page).
  auto pages_for = [&](int kb) {
    const int p_hi = (kb * 32 + 31) >> psh;
    while (p_hi >= page_base + 64) {  // uniform over the wave; once in 64 pages
      page_base += 64;
      my_page = next_pages;
      next_pages = table[min(page_base + 64 + lane, last_page)];
    }
  };
  auto load_k = [&](KVBlock& blk, int kb) {
    const int key_base = kb * 32;
    pages_for(kb);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = min(max(key_base + t * 16 + c, wlo), whi - 1);
      const int page = page_of(key);
      const bf16_t* krow = kbase + (((size_t)page * kv_row) << psh) + (size_t)(key & pmask) * HD;
      if (WIDE) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) blk.kw[t * NQ + i] = ld<NT>(reinterpret_cast<const bf16x8*>(krow + i * 32));
      } else {
#pragma unroll
        for (int i = 0; i < NQ; ++i) blk.kn[t * NQ + i] = ld<NT>(reinterpret_cast<const s16x4*>(krow + i * 16));
      }
    }
  };
  auto load_v = [&](KVBlock& blk, int kb) {
    const int key_base = kb * 32;
    pages_for(kb);
    // Slot 8 g + j of the second product holds key key_base + 4 g + j for j < 4 and key_base + 16 + 4 g + (j - 4)
    // for j >= 4, in both operands.
    const int k0 = min(max(key_base + g * 4, qlo), qhi);
    const int k1 = min(max(key_base + 16 + g * 4, qlo), qhi);
    const bf16_t* v0 = vbase + (((size_t)page_of(k0) * kv_row) << psh) + (k0 & pmask);
    const bf16_t* v1 = vbase + (((size_t)page_of(k1) * kv_row) << psh) + (k1 & pmask);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      blk.v[dt][0] = ld<NT>(reinterpret_cast<const bf16x4*>(v0 + dt * v_step));
      blk.v[dt][1] = ld<NT>(reinterpret_cast<const bf16x4*>(v1 + dt * v_step));
    }
  };
  auto load = [&](KVBlock& blk, int kb) {
    load_k(blk, kb);
    load_v(blk, kb);
  };

  // The three phases of a block: scores S^T = K Q^T; soft-max weights of the block (and the rescaling of what has been
  // summed so far); O^T += V^T P^T.
  auto scores = [&](const KVBlock& blk, f32x4 (&s)[QT][2]) {
#pragma unroll
    for (int u = 0; u < QT; ++u)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        if (WIDE) {
#pragma unroll
          for (int i = 0; i < NQ; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.kw[t * NQ + i], qw[u][i], acc, 0, 0, 0);
        } else {
#pragma unroll
          for (int i = 0; i < NQ; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(blk.kn[t * NQ + i], qn[u][i], acc, 0, 0, 0);
        }
        s[u][t] = acc;
      }
  };
  auto soften = [&](f32x4 (&s)[QT][2], int kb, bf16x8 (&pf)[QT]) {
    const int key_base = kb * 32;
    // every key of the block is seen by every column: no masks needed (uniform over the wave)
    const bool full = key_base + 31 <= full_hi && key_base >= full_lo;
#pragma unroll
    for (int u = 0; u < QT; ++u) {
      // s[u][t][j] is key key_base + 16 t + 4 g + j of column c
      float mx = -INFINITY;
      // m[u] is the running maximum of the raw scores (the scale is positive); p = 2^((s - m) scale log2 e)
      if (full) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) mx = fmaxf(mx, s[u][t][j]);
      } else {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int key = key_base + t * 16 + g * 4 + j;
            const float v = (key >= lo[u] && key <= pos[u]) ? s[u][t][j] : -INFINITY;
            s[u][t][j] = v;
            mx = fmaxf(mx, v);
          }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m[u], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const bool moved = m_new != m[u];
      const float alpha = fast_exp2((m[u] - m_safe) * a.scale_log2);
      const float shift = -m_safe * a.scale_log2;
      m[u] = m_new;
      float psum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float p = fast_exp2(fmaf(s[u][t][j], a.scale_log2, shift));
          psum += p;
          pf[u][t * 4 + j] = (bf16_t)p;
        }
      if (__any(moved)) {  // the maximum settles early in long rows; rescaling is skipped from then on
        lsum[u] *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int j = 0; j < 4; ++j) o[u][dt][j] *= alpha;
      }
      lsum[u] += psum;
    }
  };
  auto weigh = [&](const KVBlock& blk, const bf16x8 (&pf)[QT]) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const bf16x4 lo4 = blk.v[dt][0], hi4 = blk.v[dt][1];
      const bf16x8 vf = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
#pragma unroll
      for (int u = 0; u < QT; ++u) o[u][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[u], o[u][dt], 0, 0, 0);
    }
  };
  auto compute = [&](const KVBlock& blk, int kb) {
    f32x4 s[QT][2];
    bf16x8 pf[QT];
    scores(blk, s);
    soften(s, kb, pf);
    weigh(blk, pf);
  };

  constexpr int KSTEP = COOP ? 4 : 1;  // blocks between two blocks of this wave
  if (PREFETCH) {
    KVBlock ba, bb;
    int kb = kb0 + (COOP ? wave : 0);
    if (kb < kb1) load(ba, kb);
    while (kb + KSTEP < kb1) {
      load(bb, kb + KSTEP);
      compute(ba, kb);
      if (kb + 2 * KSTEP < kb1) load(ba, kb + 2 * KSTEP);
      compute(bb, kb + KSTEP);
      kb += 2 * KSTEP;
    }
    if (kb < kb1) compute(ba, kb);
  } else {
    // One set of registers, two loads in flight: the values of a block are asked for before its scores are formed, and
    // the keys of the next block as soon as the scores have read this block's keys.
    KVBlock ba;
    if (kb0 < kb1) load_k(ba, kb0);
    for (int kb = kb0; kb < kb1; ++kb) {
      f32x4 s[QT][2];
      bf16x8 pf[QT];
      load_v(ba, kb);
      scores(ba, s);
      if (kb + 1 < kb1) load_k(ba, kb + 1);
      soften(s, kb, pf);
      weigh(ba, pf);
    }
  }

  if constexpr (COOP) {
    // Lane l of every wave holds the same columns and channels, so the waves' results are joined lane by lane:
    // o = sum_w o_w 2^((m_w - m*) scale), likewise the sums, m* = max_w m_w; waves are added in order by wave 0.
    __shared__ float co[4][DT][64][4];
    __shared__ float cml[4][2][64];
    static_assert(QT == 1, "cooperative waves hold one tile");
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(co[wave][dt][lane]) = o[0][dt];
    cml[wave][0][lane] = m[0];
    cml[wave][1][lane] = lsum[0];
    __syncthreads();
    if (wave != 0) return;
    float mstar = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) mstar = fmaxf(mstar, cml[w][0][lane]);
    const float msafe = mstar == -INFINITY ? 0.f : mstar;
    float l = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[0][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float wgt = fast_exp2((cml[w][0][lane] - msafe) * a.scale_log2);
      l += cml[w][1][lane] * wgt;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(co[w][dt][lane]);
#pragma unroll
        for (int j = 0; j < 4; ++j) o[0][dt][j] += v[j] * wgt;
      }
    }
    m[0] = mstar;
    lsum[0] = l;
  }

#pragma unroll
  for (int u = 0; u < QT; ++u) {
    lsum[u] += __shfl_xor(lsum[u], 16, 64);
    lsum[u] += __shfl_xor(lsum[u], 32, 64);
    if (!col_ok[u]) continue;
    const int tt = u * (16 / a.hp) + tt0;
    // o[u][dt][j] is channel 16 dt + 4 g + j of column c
    if (a.splits == 1) {
      const size_t col = (size_t)(q0 + t0 + tt) * a.heads + head;
      const float inv = 1.f / lsum[u];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        bf16x4 r = {(bf16_t)(o[u][dt][0] * inv), (bf16_t)(o[u][dt][1] * inv), (bf16_t)(o[u][dt][2] * inv), (bf16_t)(o[u][dt][3] * inv)};
        *reinterpret_cast<bf16x4*>(a.out + col * HD + dt * 16 + g * 4) = r;
      }
    } else {
      const size_t pcol = ((size_t)tile * (QT * 16 / a.hp) + tt) * a.heads + head;
      float* po = a.part_o + (pcol * a.splits + split) * HD;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(po + dt * 16 + g * 4) = o[u][dt];
      if (g == 0) {
        a.part_ml[(pcol * a.splits + split) * 2] = m[u] * a.scale_log2;  // in the exponent's units
        a.part_ml[(pcol * a.splits + split) * 2 + 1] = lsum[u];
      }
    }
  }
}

constexpr long NT_FROM_BYTES = 192L << 20;  // keys and values of a step (all layers) from which non-temporal loads pay

template <int QT, bool PREFETCH, bool COOP>
__global__ __launch_bounds__(256) void attn_mfma_kernel(AttnParams a) {
  if constexpr (QT == 1) {
    // decode tiles carry the number of keys that the step's decode rows read over all layers (the same in every tile)
    const long bytes = (long)a.tiles[5] * a.kv_heads * HD * 4;
    if (bytes >= NT_FROM_BYTES) attn_tiles<QT, PREFETCH, COOP, true>(a);
    else attn_tiles<QT, PREFETCH, COOP, false>(a);
  } else {
    attn_tiles<QT, PREFETCH, COOP, false>(a);
  }
}

// ------------------------------------------------------------------------------------------------
// Prompt portions when the head size is a multiple of 32 up to 128 and a page holds 8 tokens or more: a workgroup owns 32 tokens
// of up to four query heads of one key/value head, one head per wave.  The four waves need the same keys and values,
// so each block of 32 keys is fetched once per workgroup, a quarter by each wave, and handed round through LDS;
// the next two blocks are on their way from memory (and the page ids one block further ahead) while this one is used.
// A tile's keys are walked by two such sets of four waves at once, each taking half of the blocks; their results are
// joined in LDS at the end.  The longest tiles set the time of a causal prompt, and this halves their chain of blocks.
//   keys in LDS:   row 16 t + 4 a + b holds key 8 a + 4 t + b of the block, so that the scores a lane gets from the
//                  two 16-key products are those of keys 8 g .. 8 g + 7: the order in which it then needs the values
//   values in LDS: [channel][32 keys], as the pages hold them
// Rows are padded by 32 bytes.  A 16-byte LDS read is served for lanes 0-7 and 16-23 together (then 8-15 and 24-31, ...),
// i.e. for eight rows at two neighbouring 16-byte columns: with rows of 2 HD + 32 and 96 bytes these sixteen pieces fall
// into sixteen different groups of four banks (the bank-conflict counter reads zero; with 16 bytes of padding every read
// took twice as long).
// ------------------------------------------------------------------------------------------------
// The largest of a value over lanes l, l ^ 16, l ^ 32 and l ^ 48, in all four of them, by the lane-swap instructions of
// gfx950: swap(a, b) exchanges the upper half of a with the lower half of b (32 lanes), or the odd 16-lane rows of a with
// the even rows of b; with a = b = x the two results hold a lane's own value and its partner's.  No LDS round trip.
__device__ __forceinline__ float max_over_lane_rows(float x) {
  const unsigned u = __float_as_uint(x);
  const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const float m = fmaxf(__uint_as_float(h[0]), __uint_as_float(h[1]));
  const unsigned v = __float_as_uint(m);
  const auto q = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  return fmaxf(__uint_as_float(q[0]), __uint_as_float(q[1]));
}

// In a stretch of straight code: N times one matrix instruction and then V vector instructions, in that order of issue.
#ifndef NS_VALU_PER_MFMA
#define NS_VALU_PER_MFMA 5
#endif
#define NS_STAGE(N, V)                                        \
  _Pragma("unroll") for (int sg_ = 0; sg_ < (N); ++sg_) {     \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        \
    __builtin_amdgcn_sched_group_barrier(0x002, (V), 0);      \
  }

constexpr bool SHARED_OK = WIDE && PS >= 8 && HD <= 128;  // larger heads do not fit two waves' registers per SIMD
constexpr int KROW = HD + 16;               // elements of a key's row in LDS
constexpr int VROW = 32 + 16;               // elements of a channel's row in LDS
constexpr int CHUNKS = 32 * HD / 8;        // 16-byte pieces of a block's keys; as many of its values
constexpr int PER_THREAD = (CHUNKS + 255) / 256;
constexpr int CPR = PS / 8 < 4 ? PS / 8 : 4;  // 16-byte pieces of a block that lie side by side in a channel's row of a page

// Two waves per SIMD: with more registers the compiler parks the sums in accumulation registers and moves them to and
// fro around every rescaling.
// SETS = 1: one set of four waves per workgroup, which walks all blocks of its range of the tile's keys.  Two such
// workgroups share a compute unit and each has a barrier of its own, so the two waves of a SIMD are not kept in the same
// phase and one's matrix instructions run under the other's soft-max arithmetic.  It pays where the ranges are joined by
// the second kernel anyway or the keys are many (the join costs a pass over the unnormalised sums).
template <int SETS>
__global__ __launch_bounds__(SETS * 256) __attribute__((amdgpu_waves_per_eu(2))) void attn_prefill_kernel(AttnParams a) {
  if constexpr (SHARED_OK) {
    constexpr int K_BYTES = 32 * KROW * 2, V_BYTES = HD * VROW * 2, SET_BYTES = 2 * (K_BYTES + V_BYTES);
    constexpr int JOIN_BYTES = SETS == 2 ? 256 * (2 * DT * 4 + 4) * 4 : 0;  // what the second set hands to the first: sums, maxima, totals
    __shared__ __align__(16) char smem[SETS * SET_BYTES > JOIN_BYTES ? SETS * SET_BYTES : JOIN_BYTES];
    // What is the same in all lanes of a wave is said to be so (readfirstlane): the loop's branches and the address
    // arithmetic that depends on the block alone then run on the scalar unit, and no branch is taken under a lane mask.
    const int half = SETS == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 8) : 0;  // which set of four waves, i.e. which half of the tile's blocks
    bf16_t(*lk)[32 * KROW] = reinterpret_cast<bf16_t(*)[32 * KROW]>(smem + half * SET_BYTES);
    bf16_t(*lv)[HD * VROW] = reinterpret_cast<bf16_t(*)[HD * VROW]>(smem + half * SET_BYTES + 2 * K_BYTES);
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, g = lane >> 4;
    const int G = a.heads / a.kv_heads;
    const int hblks = (G + 3) / 4;
    const int ny = a.kv_heads * hblks;
    const int split = blockIdx.x % a.splits, ts = blockIdx.x / a.splits;  // the ranges of a tile start together
    // Workgroups go round the eight XCDs in the order of blockIdx.x, and each XCD has an L2 of its own.  The key/value
    // head is the fast index, so with eight of them (or a divisor of eight) an XCD only ever sees one head's keys and
    // values, and every tile of a prompt re-reads them from that XCD's L2.
    const int y = ts % ny;
    // tiles are listed in the order of the tokens; the last ones see the most keys, so they start first
    const int tile = a.n_tiles - 1 - ts / ny;
    const int kvh = y / hblks, hin = (y % hblks) * 4 + wave;
    const bool head_ok = hin < G;  // a wave without a head still fetches its share of the keys and values
    const int head = kvh * G + (head_ok ? hin : 0);
    const int4 info = *reinterpret_cast<const int4*>(a.tiles + (size_t)tile * TILE_INTS);
    const int b = __builtin_amdgcn_readfirstlane(info.x), t0 = __builtin_amdgcn_readfirstlane(info.y);
    const int q0 = __builtin_amdgcn_readfirstlane(info.z), n = __builtin_amdgcn_readfirstlane(info.w);
    const int kv_len = __builtin_amdgcn_readfirstlane(a.tiles[(size_t)tile * TILE_INTS + 4]);
    const int* table = a.block_table + (size_t)b * a.table_stride;
    constexpr int psh = __builtin_ctz(PS), pmask = PS - 1;

    bool col_ok[2];
    int pos[2], lo[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int ti = t0 + u * 16 + c;
      col_ok[u] = ti < n && head_ok;
      pos[u] = col_ok[u] ? kv_len - n + ti : -1;
      lo[u] = (col_ok[u] && a.window > 0) ? max(0, pos[u] - a.window + 1) : 0;
    }
    // what the tile's tokens see, from the descriptor alone: the same in every wave
    const int first_pos = kv_len - n + t0, last_pos = kv_len - n + min(t0 + 31, n - 1);
    const int whi = last_pos + 1;                                                   // keys [wlo, whi) are seen by some token
    const int wlo = a.window > 0 ? max(0, first_pos - a.window + 1) : 0;
    const int full_hi = first_pos;                                                  // keys <= full_hi are seen by every token
    const int full_lo = a.window > 0 ? max(0, last_pos - a.window + 1) : 0;         // ... if they are >= full_lo
    int tile_kb0 = wlo / 32, tile_kb1 = (whi + 31) / 32;
    if (a.splits > 1) {  // this workgroup's range of the tile's blocks; it may be empty
      const int per = (tile_kb1 - tile_kb0 + a.splits - 1) / a.splits;
      tile_kb0 = min(tile_kb1, tile_kb0 + split * per);
      tile_kb1 = min(tile_kb1, tile_kb0 + per);
    }
    const int steps = SETS == 2 ? (tile_kb1 - tile_kb0 + 1) / 2 : tile_kb1 - tile_kb0;  // blocks of the first set; the second has as many or one fewer
    const int kb0 = half ? tile_kb0 + steps : tile_kb0, kb1 = (half || SETS == 1) ? tile_kb1 : tile_kb0 + steps;

    bf16x8 qw[2][NQ];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int ti = t0 + u * 16 + c;
      const bf16_t* qrow = a.q + (size_t)(q0 + (col_ok[u] ? ti : 0)) * a.q_stride + head * HD;
#pragma unroll
      for (int i = 0; i < NQ; ++i) {
        qw[u][i] = *reinterpret_cast<const bf16x8*>(qrow + i * 32 + g * 8);
        if (!col_ok[u]) qw[u][i] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
    f32x4 o[2][DT];
    float m[2], lsum[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      m[u] = -INFINITY;
      lsum[u] = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[u][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    const bf16_t one = (bf16_t)1.0f;
    const bf16x8 ones = {one, one, one, one, one, one, one, one};
    // This thread's pieces of a block: piece r of the keys is 8 channels of one key, piece r of the values 8 keys of
    // one channel.
    int k_key[PER_THREAD], k_off[PER_THREAD], k_lds[PER_THREAD];
    int v_kq[PER_THREAD], v_ch[PER_THREAD], v_lds[PER_THREAD];
    bool mine[PER_THREAD];
#pragma unroll
    for (int r = 0; r < PER_THREAD; ++r) {
      const int qi = tid + 256 * r;
      mine[r] = qi < CHUNKS;
      const int q = mine[r] ? qi : 0;
      const int key = q / (HD / 8), piece = q % (HD / 8);
      k_key[r] = key;
      k_off[r] = piece * 8;
      k_lds[r] = (16 * ((key & 7) >> 2) + 4 * (key >> 3) + (key & 3)) * KROW + piece * 8;
      const int pg = q / (CPR * HD), rem = q % (CPR * HD);
      v_ch[r] = rem / CPR;
      v_kq[r] = pg * CPR + rem % CPR;
      v_lds[r] = v_ch[r] * VROW + v_kq[r] * 8;
    }
    const int vlo = wlo & ~7, vhi = (whi - 1) & ~7;
    const size_t k_head = ((size_t)kvh * HD) << psh, kv_page = ((size_t)a.kv_heads * HD) << psh;  // elements
    // A block that lies wholly inside [wlo, whi) and pages that divide a block: page slots and offsets inside a page
    // are the same in every block, up to the block's first slot.
    constexpr bool EVEN = PS <= 32;
    constexpr int PPB = EVEN ? 32 / PS : 1;  // pages per block
    int k_slot[PER_THREAD], v_slot[PER_THREAD], k_const[PER_THREAD], v_const[PER_THREAD];
#pragma unroll
    for (int r = 0; r < PER_THREAD; ++r) {
      k_slot[r] = k_key[r] >> psh;
      v_slot[r] = (v_kq[r] * 8) >> psh;
      k_const[r] = (int)k_head + (k_key[r] & pmask) * HD + k_off[r];
      v_const[r] = (int)k_head + (v_ch[r] << psh) + ((v_kq[r] * 8) & pmask);
    }
    auto inside = [&](int kb) { return EVEN && kb * 32 >= wlo && kb * 32 + 31 < whi; };
    // Two blocks are on their way from memory at a time (a block's compute is shorter than the latency of its loads):
    // register set (kb - kb0) & 1 holds block kb between its loads and its copy into LDS, and the page ids of block kb
    // from a round before its loads.  Loads return in the order of issue, so a round asks for the next page ids before
    // it asks for keys and values: waiting for those page ids a round later then leaves the keys and values in flight.
    int kps[2][PER_THREAD], vps[2][PER_THREAD];
    bf16x8 kst[2][PER_THREAD], vst[2][PER_THREAD];
    // Otherwise addresses are kept inside held pages: a key outside [wlo, whi) is masked anyway.
    auto fetch_pages = [&](int(&kp)[PER_THREAD], int(&vp)[PER_THREAD], int kb) {
      const bool in = inside(kb);
#pragma unroll
      for (int r = 0; r < PER_THREAD; ++r) {  // one load each, from an index chosen beforehand
        const int ks = in ? kb * PPB + k_slot[r] : min(max(kb * 32 + k_key[r], wlo), whi - 1) >> psh;
        const int vs = in ? kb * PPB + v_slot[r] : min(max(kb * 32 + v_kq[r] * 8, vlo), vhi) >> psh;
        kp[r] = table[ks];
        vp[r] = table[vs];
      }
    };
    auto fetch = [&](bf16x8(&kr)[PER_THREAD], bf16x8(&vr)[PER_THREAD], const int(&kp)[PER_THREAD], const int(&vp)[PER_THREAD], int kb) {
      if (inside(kb)) {
#pragma unroll
        for (int r = 0; r < PER_THREAD; ++r) {
          kr[r] = *reinterpret_cast<const bf16x8*>(a.k_cache + (size_t)kp[r] * kv_page + k_const[r]);
          vr[r] = *reinterpret_cast<const bf16x8*>(a.v_cache + (size_t)vp[r] * kv_page + v_const[r]);
        }
      } else {
#pragma unroll
        for (int r = 0; r < PER_THREAD; ++r) {
          const int key = min(max(kb * 32 + k_key[r], wlo), whi - 1);
          kr[r] = *reinterpret_cast<const bf16x8*>(a.k_cache + (size_t)kp[r] * kv_page + k_head + (size_t)(key & pmask) * HD + k_off[r]);
          const int key8 = min(max(kb * 32 + v_kq[r] * 8, vlo), vhi);
          vr[r] = *reinterpret_cast<const bf16x8*>(a.v_cache + (size_t)vp[r] * kv_page + k_head + ((size_t)v_ch[r] << psh) + (key8 & pmask));
        }
      }
    };
    auto put = [&](const bf16x8(&kr)[PER_THREAD], const bf16x8(&vr)[PER_THREAD], int buf) {
#pragma unroll
      for (int r = 0; r < PER_THREAD; ++r)
        if (mine[r]) {
          *reinterpret_cast<bf16x8*>(&lk[buf][k_lds[r]]) = kr[r];
          *reinterpret_cast<bf16x8*>(&lv[buf][v_lds[r]]) = vr[r];
        }
    };

    // One block of 32 keys for this wave's two 16-token columns.  The order of the source is the order of issue: the
    // matrix instructions of one column run while the vector unit does the soft-max arithmetic of the other
    // (scores u0, scores u1 | soft-max u0 under them, sums u0 | soft-max u1 under them, sums u1).
    auto block = [&](int buf, int kb, auto full_tag) {
      // full_tag: every key of the block is seen by every token of the tile (known when the loop was entered), so the
      // code of such blocks holds no masks at all; the few blocks at the ends of a tile's keys run the other form
      constexpr bool FULL = decltype(full_tag)::value;
      const int key_base = kb * 32;
      bf16x8 kf[2][NQ];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < NQ; ++i) kf[t][i] = *reinterpret_cast<const bf16x8*>(&lk[buf][(16 * t + c) * KROW + 32 * i + 8 * g]);
      f32x4 s[2][2];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < NQ; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][i], qw[u][i], acc, 0, 0, 0);
          s[u][t] = acc;
        }
      // s[u][t][j] is key key_base + 8 g + 4 t + j of column c
      bf16x8 pf[2];
      auto soften = [&](int u) {
        float mx = -INFINITY;
        if (!FULL) {
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int key = key_base + g * 8 + t * 4 + j;
              s[u][t][j] = (key >= lo[u] && key <= pos[u]) ? s[u][t][j] : -INFINITY;
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) mx = fmaxf(mx, s[u][t][j]);
        mx = max_over_lane_rows(mx);
        // m[u] is the running maximum of the raw scores (the scale is positive); p = 2^((s - m) scale log2 e)
        const float m_new = fmaxf(m[u], mx);
        const float m_safe = (!FULL && m_new == -INFINITY) ? 0.f : m_new;  // (a full block's maximum is a score)
        const bool moved = m_new != m[u];
        const float alpha = fast_exp2((m[u] - m_safe) * a.scale_log2);
        const float shift = -m_safe * a.scale_log2;
        m[u] = m_new;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) pf[u][t * 4 + j] = (bf16_t)fast_exp2(fmaf(s[u][t][j], a.scale_log2, shift));
        if (__any(moved)) {  // the maximum settles early in long rows; rescaling is skipped from then on
          lsum[u] *= alpha;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int j = 0; j < 4; ++j) o[u][dt][j] *= alpha;
        }
      };
#ifdef NS_VONCE
      bf16x8 vfr[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vfr[dt] = *reinterpret_cast<const bf16x8*>(&lv[buf][(16 * dt + c) * VROW + 8 * g]);
#endif
      auto weigh = [&](int u) {
        // the block's sum of weights by one more matrix instruction against ones: every row of the result is the sum over
        // the 32 keys of the weights as the value products see them (rounded to bfloat16), for this lane's column
        const f32x4 tot = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pf[u], f32x4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#ifdef NS_VONCE
          const bf16x8 vf = vfr[dt];
#else
          const bf16x8 vf = *reinterpret_cast<const bf16x8*>(&lv[buf][(16 * dt + c) * VROW + 8 * g]);
#endif
          o[u][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[u], o[u][dt], 0, 0, 0);
        }
        lsum[u] += tot[0];
      };
      soften(0);
      weigh(0);
      soften(1);
      weigh(1);
    };

    // Before round it: block kb0 + it lies in LDS buffer it & 1, block kb0 + it + 1 is on its way into register set
    // (it + 1) & 1, and the page ids of block kb0 + it + 2 are on their way into page set it & 1.
    if (kb0 < kb1) {
      fetch_pages(kps[0], vps[0], kb0);
      if (kb0 + 1 < kb1) fetch_pages(kps[1], vps[1], kb0 + 1);
      fetch(kst[0], vst[0], kps[0], vps[0], kb0);
      if (kb0 + 1 < kb1) {
        if (kb0 + 2 < kb1) fetch_pages(kps[0], vps[0], kb0 + 2);  // set 0 is free once block kb0's loads are issued
        fetch(kst[1], vst[1], kps[1], vps[1], kb0 + 1);
      }
      put(kst[0], vst[0], 0);
    }
    __syncthreads();
    // One round: the page ids of block it + 3 and then the keys and values of block it + 2 are asked for, this block is
    // used, and the next block goes from its registers (loaded a round ago) into the other LDS buffer.  Both sets pass
    // every barrier; the second may have no block in the last round.
    auto round = [&](bf16x8(&kr_far)[PER_THREAD], bf16x8(&vr_far)[PER_THREAD], int(&kp_far)[PER_THREAD], int(&vp_far)[PER_THREAD],
                     const bf16x8(&kr_next)[PER_THREAD], const bf16x8(&vr_next)[PER_THREAD], int(&kp_next)[PER_THREAD],
                     int(&vp_next)[PER_THREAD], int it, auto full_tag) {
      const int kb = kb0 + it;
      const int buf = it & 1;
      if (kb + 2 < kb1) {
        if (kb + 3 < kb1) fetch_pages(kp_next, vp_next, kb + 3);  // the set that block it + 1's loads were issued from
        fetch(kr_far, vr_far, kp_far, vp_far, kb + 2);
      }
      if (head_ok && kb < kb1) block(buf, kb, full_tag);
      if (kb + 1 < kb1) put(kr_next, vr_next, buf ^ 1);
      __syncthreads();
    };
    // A round of the long middle of a tile's keys, where nothing needs asking: the block is seen wholly by every token, all
    // four waves have a head, and the blocks whose ids and data are asked for lie inside the tile's keys and are not the
    // last.  Its matrix instructions and its vector arithmetic are laid side by side, stage by stage, because the matrix
    // unit runs a wave's instruction while the wave issues vector instructions that do not wait for it:
    //   1  the next loads are issued               beside  the scores of the first column
    //   2  the first column's soft-max weights     beside  the scores of the second column
    //   3  the second column's soft-max weights    beside  the first column's weighted values
    //   4  the next block goes into LDS            beside  the second column's weighted values
    // (a column's sums are rescaled between two stages, and only when its maximum moved).
    auto steady = [&](bf16x8(&kr_far)[PER_THREAD], bf16x8(&vr_far)[PER_THREAD], int(&kp_far)[PER_THREAD], int(&vp_far)[PER_THREAD],
                      const bf16x8(&kr_next)[PER_THREAD], const bf16x8(&vr_next)[PER_THREAD], int(&kp_next)[PER_THREAD],
                      int(&vp_next)[PER_THREAD], int it, auto near_tag) {
      constexpr bool NEAR = decltype(near_tag)::value;
      const int kb = kb0 + it, buf = it & 1;
      const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
      // ---- 1
#pragma unroll
      for (int r = 0; r < PER_THREAD; ++r) {
        kp_next[r] = table[(kb + 3) * PPB + k_slot[r]];
        vp_next[r] = table[(kb + 3) * PPB + v_slot[r]];
      }
#pragma unroll
      for (int r = 0; r < PER_THREAD; ++r) {
        if (NEAR) {
          const unsigned page_bytes = (unsigned)kv_page * 2;
          const unsigned ko = __umul24((unsigned)kp_far[r], page_bytes) + (unsigned)k_const[r] * 2;
          const unsigned vo = __umul24((unsigned)vp_far[r], page_bytes) + (unsigned)v_const[r] * 2;
          kr_far[r] = *reinterpret_cast<const bf16x8*>(reinterpret_cast<const char*>(a.k_cache) + ko);
          vr_far[r] = *reinterpret_cast<const bf16x8*>(reinterpret_cast<const char*>(a.v_cache) + vo);
        } else {
          kr_far[r] = *reinterpret_cast<const bf16x8*>(a.k_cache + (size_t)kp_far[r] * kv_page + k_const[r]);
          vr_far[r] = *reinterpret_cast<const bf16x8*>(a.v_cache + (size_t)vp_far[r] * kv_page + v_const[r]);
        }
      }
      bf16x8 kf[2][NQ];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < NQ; ++i) kf[t][i] = *reinterpret_cast<const bf16x8*>(&lk[buf][(16 * t + c) * KROW + 32 * i + 8 * g]);
      f32x4 s[2][2];
      auto scores = [&](int u) {
#pragma unroll
        for (int t = 0; t < 2; ++t) s[u][t] = zero4;
#pragma unroll
        for (int i = 0; i < NQ; ++i)
#pragma unroll
          for (int t = 0; t < 2; ++t) s[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][i], qw[u][i], s[u][t], 0, 0, 0);
      };
      bf16x8 pf[2];
      float alpha[2];
      auto soften = [&](int u) -> bool {
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) mx = fmaxf(mx, s[u][t][j]);
        mx = max_over_lane_rows(mx);
        const float m_new = fmaxf(m[u], mx);
        const bool moved = m_new != m[u];
        alpha[u] = fast_exp2((m[u] - m_new) * a.scale_log2);
        const float shift = -m_new * a.scale_log2;
        m[u] = m_new;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) pf[u][t * 4 + j] = (bf16_t)fast_exp2(fmaf(s[u][t][j], a.scale_log2, shift));
        return __any(moved);
      };
      auto rescale = [&](int u) {
        lsum[u] *= alpha[u];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int j = 0; j < 4; ++j) o[u][dt][j] *= alpha[u];
      };
      auto weigh = [&](int u) {
        const f32x4 tot = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pf[u], zero4, 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const bf16x8 vf = *reinterpret_cast<const bf16x8*>(&lv[buf][(16 * dt + c) * VROW + 8 * g]);
          o[u][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[u], o[u][dt], 0, 0, 0);
        }
        lsum[u] += tot[0];
      };
      scores(0);
      __builtin_amdgcn_sched_barrier(0);
      // ---- 2
      scores(1);
      const bool moved0 = soften(0);
      NS_STAGE(8, NS_VALU_PER_MFMA)
      asm volatile("" : "+v"(pf[0]));  // the weights are formed here, beside the matrix instructions, not where they are used
      __builtin_amdgcn_sched_barrier(0);
      if (moved0) rescale(0);
      // ---- 3
      weigh(0);
      const bool moved1 = soften(1);
      NS_STAGE(9, NS_VALU_PER_MFMA)
      asm volatile("" : "+v"(pf[1]));
      __builtin_amdgcn_sched_barrier(0);
      if (moved1) rescale(1);
      // ---- 4
      weigh(1);
#pragma unroll
      for (int r = 0; r < PER_THREAD; ++r)
        if (mine[r]) {
          *reinterpret_cast<bf16x8*>(&lk[buf ^ 1][k_lds[r]]) = kr_next[r];
          *reinterpret_cast<bf16x8*>(&lv[buf ^ 1][v_lds[r]]) = vr_next[r];
        }
      __syncthreads();
    };

    // The first blocks of this set's range that every token of the tile sees wholly (an even number of them: rounds go in
    // pairs, one per register set) run the form without masks.  Both sets pass a barrier in every round, whichever form
    // a round takes.
    const int seen_whole = a.window > 0 ? 0 : min(max((full_hi + 1) / 32 - kb0, 0), max(kb1 - kb0, 0)) & ~1;
    const bool all_heads = (y % hblks) * 4 + 3 < G;
    const int n_steady = (EVEN && all_heads) ? max(min(seen_whole, kb1 - kb0 - 4), 0) & ~1 : 0;
    int it = 0;
    if (a.near) {
      for (; it < n_steady; it += 2) {
        steady(kst[0], vst[0], kps[0], vps[0], kst[1], vst[1], kps[1], vps[1], it, std::true_type{});
        steady(kst[1], vst[1], kps[1], vps[1], kst[0], vst[0], kps[0], vps[0], it + 1, std::true_type{});
      }
    } else {
      for (; it < n_steady; it += 2) {
        steady(kst[0], vst[0], kps[0], vps[0], kst[1], vst[1], kps[1], vps[1], it, std::false_type{});
        steady(kst[1], vst[1], kps[1], vps[1], kst[0], vst[0], kps[0], vps[0], it + 1, std::false_type{});
      }
    }
    for (; it < seen_whole; it += 2) {
      round(kst[0], vst[0], kps[0], vps[0], kst[1], vst[1], kps[1], vps[1], it, std::true_type{});
      round(kst[1], vst[1], kps[1], vps[1], kst[0], vst[0], kps[0], vps[0], it + 1, std::true_type{});
    }
    for (; it < steps; it += 2) {
      round(kst[0], vst[0], kps[0], vps[0], kst[1], vst[1], kps[1], vps[1], it, std::false_type{});
      if (it + 1 < steps) round(kst[1], vst[1], kps[1], vps[1], kst[0], vst[0], kps[0], vps[0], it + 1, std::false_type{});
    }

    // The second set hands its sums to the first, lane by lane (both hold the same columns and channels):
    // o = o_0 2^((m_0 - m*) scale) + o_1 2^((m_1 - m*) scale), likewise the totals, m* = max(m_0, m_1).
    float* join = reinterpret_cast<float*>(smem) + tid * (2 * DT * 4 + 4);
    if (SETS == 2 && half) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(join + (u * DT + dt) * 4) = o[u][dt];
        join[2 * DT * 4 + u] = m[u];
        join[2 * DT * 4 + 2 + u] = lsum[u];
      }
    }
    if (SETS == 2) __syncthreads();
    if (half) return;
#pragma unroll
    for (int u = 0; SETS == 2 && u < 2; ++u) {
      const float m1 = join[2 * DT * 4 + u], l1 = join[2 * DT * 4 + 2 + u];
      const float mstar = fmaxf(m[u], m1);
      const float msafe = mstar == -INFINITY ? 0.f : mstar;
      const float w0 = fast_exp2((m[u] - msafe) * a.scale_log2), w1 = fast_exp2((m1 - msafe) * a.scale_log2);
      lsum[u] = lsum[u] * w0 + l1 * w1;
      m[u] = mstar;  // what the sums now refer to: a range's maximum goes out with them
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(join + (u * DT + dt) * 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) o[u][dt][j] = o[u][dt][j] * w0 + v[j] * w1;
      }
    }

#pragma unroll
    for (int u = 0; u < 2; ++u) {
      // (lsum[u] is the column's whole sum in every lane of the column: the matrix instruction added over all keys)
      if (!col_ok[u]) continue;
      // o[u][dt][j] is channel 16 dt + 4 g + j of column c
      if (a.splits == 1) {
        const size_t col = (size_t)(q0 + t0 + u * 16 + c) * a.heads + head;
        const float inv = 1.f / lsum[u];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          bf16x4 r = {(bf16_t)(o[u][dt][0] * inv), (bf16_t)(o[u][dt][1] * inv), (bf16_t)(o[u][dt][2] * inv), (bf16_t)(o[u][dt][3] * inv)};
          *reinterpret_cast<bf16x4*>(a.out + col * HD + dt * 16 + g * 4) = r;
        }
      } else {  // as the ranges of a decode tile: unnormalised sums, maximum in the exponent's units, total
        const size_t pcol = ((size_t)tile * 32 + u * 16 + c) * a.heads + head;
        float* po = a.part_o + (pcol * a.splits + split) * HD;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f32x4*>(po + dt * 16 + g * 4) = o[u][dt];
        if (g == 0) {
          a.part_ml[(pcol * a.splits + split) * 2] = m[u] * a.scale_log2;
          a.part_ml[(pcol * a.splits + split) * 2 + 1] = lsum[u];
        }
      }
    }
  }
}

#include "attn_prefill32.h"

// Joining the key ranges: out[col] = sum_s o_s 2^(m_s - m*) / sum_s l_s 2^(m_s - m*), m* = max_s m_s.
// One wave per (tile, token of the tile, head); lane s first holds range s (at most 64 ranges), so the maxima and
// weights are formed by wave reductions, then the lanes split the channels and add the ranges in order.  The ranges'
// results are addressed by tile, so nothing here waits for the tile descriptor except the final store.
__global__ __launch_bounds__(64) void attn_reduce_kernel(bf16_t* __restrict__ out, const float* __restrict__ part_o,
                                                         const float* __restrict__ part_ml, const int* __restrict__ tiles,
                                                         int heads, int tile_tokens, int splits) {
  const int tile = blockIdx.x, head = blockIdx.y, tt = blockIdx.z;
  const int lane = threadIdx.x;
  const size_t pcol = ((size_t)tile * tile_tokens + tt) * heads + head;
  const float* ml = part_ml + pcol * splits * 2;
  float ms = -INFINITY, ls = 0.f;
  if (lane < splits) {
    ms = ml[lane * 2];
    ls = ml[lane * 2 + 1];
  }
  constexpr int PER = (HD + 63) / 64;
  const float* po = part_o + pcol * splits * HD;
  const int4 info = *reinterpret_cast<const int4*>(tiles + (size_t)tile * TILE_INTS);
  const int ti = info.y + tt;
  if (ti >= info.w) return;  // the tile holds fewer tokens
  float mstar = ms;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mstar = fmaxf(mstar, __shfl_xor(mstar, o, 64));
  const float wgt = ms == -INFINITY ? 0.f : exp2f(ms - mstar);
  float l = ls * wgt;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o, 64);
  const float inv = 1.f / l;
  float acc[PER];
#pragma unroll
  for (int p = 0; p < PER; ++p) acc[p] = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 8) {  // eight ranges' loads in flight at a time
    float v[8][PER];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int p = 0; p < PER; ++p) {
        const int d = lane + p * 64;
        v[i][p] = (s0 + i < splits && d < HD) ? po[(size_t)(s0 + i) * HD + d] : 0.f;
      }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float ws = __shfl(wgt, (s0 + i) & 63, 64);
#pragma unroll
      for (int p = 0; p < PER; ++p) acc[p] += v[i][p] * ws;
    }
  }
  const size_t col = (size_t)(info.z + ti) * heads + head;
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    const int d = lane + p * 64;
    if (d < HD) out[col * HD + d] = (bf16_t)(acc[p] * inv);
  }
}

extern "C" int ns_attn_mfma_head_dim() { return HD; }
extern "C" int ns_attn_mfma_page_size() { return PS; }

// Workspace, when splits > 1: with T = qt*16/hp tokens in a tile, part_o holds n_tiles*T*heads*splits*HD floats and
// part_ml n_tiles*T*heads*splits*2.
// Which kernel takes prompt portions in tiles of 32 tokens in this library: 32 attn_prefill32_kernel, 16
// attn_prefill_kernel, 0 attn_mfma_kernel.  attn_prefill32_kernel counts its loads by hand, so it must have no others:
// were it ever compiled with registers spilled to scratch memory (whose accesses count among the loads), the 16x16
// kernel takes its place.
static int prompt_form() {
  if (!SHARED_OK) return 0;
#ifndef NS_PREFILL16
  static const bool counts_hold = [] {
    hipFuncAttributes one, two;
    return hipFuncGetAttributes(&one, reinterpret_cast<const void*>(&attn_prefill32_kernel<1>)) == hipSuccess &&
           hipFuncGetAttributes(&two, reinterpret_cast<const void*>(&attn_prefill32_kernel<2>)) == hipSuccess && one.localSizeBytes == 0 &&
           two.localSizeBytes == 0;
  }();
  if (DMA_OK && counts_hold) return 32;
#endif
  return 16;
}
extern "C" int ns_attn_prompt_form(void) { return prompt_form(); }

extern "C" int ns_attn_mfma(void* out, void* part_o, void* part_ml, const void* q, int q_stride, const void* k_cache,
                            const void* v_cache, const int* tiles, const int* block_table, int table_stride, int n_tiles,
                            int heads, int kv_heads, int page_size, int hp, int splits, int window, float scale, int qt,
                            int coop, long pool_pages, hipStream_t stream) {
  if (n_tiles <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || page_size != PS || window < 0 ||
      splits < 1 || splits > 64 || (q_stride & 7) || ((uintptr_t)tiles & 15))
    return NS_ERR_BAD_ARG;
  if (hp != 1 && hp != 2 && hp != 4 && hp != 8 && hp != 16) return NS_ERR_BAD_ARG;
  if (!(scale > 0.f)) return NS_ERR_BAD_ARG;  // maxima are tracked on unscaled scores
  if (splits > 1 && (!part_o || !part_ml)) return NS_ERR_BAD_ARG;
  // (with qt == 2, coop asks for one set of four waves per workgroup: see attn_prefill_kernel)
  if (qt != 1 && !(qt == 2 && hp == 1)) return NS_ERR_BAD_ARG;
  AttnParams a;
  a.out = (bf16_t*)out; a.part_o = (float*)part_o; a.part_ml = (float*)part_ml;
  a.q = (const bf16_t*)q; a.k_cache = (const bf16_t*)k_cache; a.v_cache = (const bf16_t*)v_cache;
  a.tiles = tiles; a.block_table = block_table;
  a.q_stride = q_stride; a.table_stride = table_stride; a.n_tiles = n_tiles; a.heads = heads; a.kv_heads = kv_heads;
  a.hp = hp; a.splits = splits; a.window = window;
  const long page_bytes = (long)kv_heads * HD * PS * 2;
  a.near = pool_pages > 0 && pool_pages < (1L << 24) && page_bytes < (1L << 24) && pool_pages * page_bytes <= (1L << 32);
  a.scale_log2 = scale * 1.4426950408889634f;
  const int G = heads / kv_heads;
  const long items = (long)n_tiles * splits * kv_heads * ((G + hp - 1) / hp);
  const long blocks = coop ? items : (items + 3) / 4;
  if (blocks > 0x7fffffffL) return NS_ERR_BAD_ARG;
  if (qt == 2 && SHARED_OK) {
    const long wgs = (long)n_tiles * splits * kv_heads * ((G + 3) / 4);
    if (wgs > 0x7fffffffL) return NS_ERR_BAD_ARG;
#ifndef NS_PREFILL16
    if (prompt_form() == 32) {
      if (coop)
        attn_prefill32_kernel<1><<<(unsigned)wgs, 256, 0, stream>>>(a);
      else
        attn_prefill32_kernel<2><<<(unsigned)wgs, 512, 0, stream>>>(a);
    } else
#endif
    if (coop)
      attn_prefill_kernel<1><<<(unsigned)wgs, 256, 0, stream>>>(a);
    else
      attn_prefill_kernel<2><<<(unsigned)wgs, 512, 0, stream>>>(a);
  } else if (qt == 2)
    attn_mfma_kernel<2, false, false><<<(unsigned)blocks, 256, 0, stream>>>(a);
  else if (coop)
    attn_mfma_kernel<1, true, true><<<(unsigned)blocks, 256, 0, stream>>>(a);
  else
    attn_mfma_kernel<1, true, false><<<(unsigned)blocks, 256, 0, stream>>>(a);
  const int st = ns_launch_status();
  if (st != NS_OK || splits == 1) return st;
  if (heads > 65535) return NS_ERR_BAD_ARG;
  const int tile_tokens = qt * 16 / hp;
  attn_reduce_kernel<<<dim3(n_tiles, heads, tile_tokens), 64, 0, stream>>>((bf16_t*)out, (const float*)part_o, (const float*)part_ml,
                                                                           tiles, heads, tile_tokens, splits);
  return ns_launch_status();
}
