// Rotary position encoding, in one place for every kernel that applies it: the stand-alone rotation kernels
// (elementwise.hip), the kernel that joins the ranges of a q/k/v product (elementwise.hip) and the epilogue of the
// few-row q/k/v product (gemm_bf16.hip).
//
// A head's first ``rot`` channels are rotated in pairs; pair j turns by angle = position * inv_freq[j], formed in
// 32-bit (reference: model/llama.py:133-136):
//     a' = a cos - b sin ;  b' = b cos + a sin                       (reference: model/llama.py:150-158)
// Which two channels make pair j is the form's ``interleaved``: 0 pairs channel j with j + rot/2 (the reference's
// half-split form), 1 pairs 2j with 2j + 1.  ``factor`` multiplies cosine and sine (1 leaves them as they are, exactly).
#pragma once
#include <hip/hip_runtime.h>
#include "common.h"

struct RopeForm {
  int rot;          // rotary channels of a head (even, at most the head size)
  int interleaved;  // pairing, see above
  float factor;     // on cosine and sine
};

// the two channels of pair j (a, b in the formula above)
__device__ __forceinline__ void rope_pair_channels(const RopeForm f, int j, int& d1, int& d2) {
  if (f.interleaved) {
    d1 = 2 * j;
    d2 = 2 * j + 1;
  } else {
    d1 = j;
    d2 = j + f.rot / 2;
  }
}

__device__ __forceinline__ void rope_cos_sin(const RopeForm f, int pos, float inv_freq, float& c, float& s) {
  const float ang = (float)pos * inv_freq;
  c = cosf(ang) * f.factor;
  s = sinf(ang) * f.factor;
}

__device__ __forceinline__ void rope_turn(float a, float b, float c, float s, float& a2, float& b2) {
  a2 = a * c - b * s;
  b2 = b * c + a * s;
}

// What the epilogue of a stacked q/k/v product needs: the rows of the stacked [q; k; v] matrix were permuted at load time
// so that a tile of 16 rows is, for the rotary part of a q or k head, the first channels of 8 pairs j and then their
// second channels (j and j + rot/2, or 2j and 2j + 1), and otherwise 16 consecutive channels.  The epilogue rotates,
// writes q into the attention input, k into its K page slot and v into the transposed V page
// (reference: model/llama.py:175-183; kv/cache.py:23-26).
struct RopeKvParams {
  const int* positions;    // [M]
  const int* token_req;    // [M]
  const int* block_table;  // [requests, table_stride]
  const float* inv_freq;   // [rot / 2]
  bf16_t* k_cache;         // [pages, kv_heads, page, hd]
  bf16_t* v_cache;         // [pages, kv_heads, hd, page]
  int table_stride, heads, kv_heads, hd, rot, page_size, write_kv;
  RopeForm form;           // rot again, the pairing and the factor on cosine and sine
};

// One pair of sums of such a product: x1, x2 are the sums of local rows p and p + 8 (p = 0 .. 7) of tile jt of head gh
// (among [q heads | k heads | v heads]) for token m.  Rotated if the tile lies in the head's rotary part, then stored:
// q into out[m][head gh], k and v into the token's slot of their pages (if write_kv).
__device__ __forceinline__ void rope_kv_store_pair(const RopeKvParams& rk, void* out, int out_stride, int m, int gh, int jt, int p,
                                                   float x1, float x2) {
  const bool is_q = gh < rk.heads, is_v = gh >= rk.heads + rk.kv_heads;
  const int rot_tiles = is_v ? 0 : rk.rot / 16;
  int d1, d2;
  if (jt < rot_tiles) {
    const int j = jt * 8 + p;
    float c, sn;
    rope_cos_sin(rk.form, rk.positions[m], rk.inv_freq[j], c, sn);
    rope_turn(x1, x2, c, sn, x1, x2);
    rope_pair_channels(rk.form, j, d1, d2);
  } else {
    d1 = rk.rot * (is_v ? 0 : 1) + (jt - rot_tiles) * 16 + p;
    d2 = d1 + 8;
  }
  if (is_q) {
    bf16_t* o = (bf16_t*)out + (size_t)m * out_stride + gh * rk.hd;
    o[d1] = (bf16_t)x1;
    o[d2] = (bf16_t)x2;
  } else if (rk.write_kv) {
    const int pos = rk.positions[m];
    const int page = rk.block_table[(size_t)rk.token_req[m] * rk.table_stride + pos / rk.page_size];
    const int off = pos % rk.page_size;
    if (!is_v) {
      const int kh = gh - rk.heads;
      bf16_t* kd = rk.k_cache + (((size_t)page * rk.kv_heads + kh) * rk.page_size + off) * rk.hd;
      kd[d1] = (bf16_t)x1;
      kd[d2] = (bf16_t)x2;
    } else {
      const int vh = gh - rk.heads - rk.kv_heads;
      bf16_t* vd = rk.v_cache + (((size_t)page * rk.kv_heads + vh) * rk.hd) * rk.page_size + off;
      vd[(size_t)d1 * rk.page_size] = (bf16_t)x1;
      vd[(size_t)d2 * rk.page_size] = (bf16_t)x2;
    }
  }
}
