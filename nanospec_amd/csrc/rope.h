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
