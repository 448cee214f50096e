// Optional terms of masked softmax attention, shared by the row kernels and
// the matrix-core prefill kernel.  For query position i and key j of head h:
//
//   s = q.k * scale
//   s <- cap * tanh(s / cap)                    (cap > 0)
//   s <- s - r1[h] * ln(1 + r2[h] * (i - j))    (r1 given)
//   softmax denominator += exp(sink[h])         (sink given: a keyless,
//                                                valueless, unscaled term)
//
// first > 0: the keys j < first stay visible to every later row whatever the
// chunk or window says (at their true positions).
//
// ldv is the row stride of the value pages in elements: dv for pages of
// their own, dk when the values are the leading dv elements of the key rows
// (vc == kc; latent attention keeps one row per token).
#pragma once
#include "common.h"

struct AttnExtra {
  const float* sink;   // [H] or null
  const float* r1;     // [H] or null
  const float* r2;     // [H] (with r1)
  float cap;           // 0: no soft cap
  i64 ldv;
  int first;           // 0: no always-visible leading keys
};

// exact forms (fp32 storage and the row kernels)
__device__ __forceinline__ float attn_softcap(float s, float cap) {
  return cap > 0.f ? cap * tanhf(s / cap) : s;
}
__device__ __forceinline__ float attn_dist_bias(float r1, float r2, int dist) {
  return r1 * logf(1.0f + r2 * (float)dist);
}
// hardware-transcendental soft cap for scores that are rounded to bf16
// weights afterwards: tanh(x) = 1 - 2 / (1 + e^(2x))
__device__ __forceinline__ float attn_softcap_fast(float s, float inv_cap, float cap) {
  const float e = __expf(2.0f * s * inv_cap);
  return cap - 2.0f * cap * __frcp_rn(1.0f + e);
}
