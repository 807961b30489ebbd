// What an attention layer may have beyond a scale, a window and a cap on its scores. All of it is off when zero or null.
//   sink        [heads] 32-bit: exp(sink[h]) joins the softmax's denominator, once; it has no key and no value
//   rel, rel_far  [heads, rel_far + 1] 32-bit: rel[h, min(i - j, rel_far)] is added to the scaled score of query
//               position i and key position j (a table by distance, made by the host from whatever the model learned)
//   keep_first  with a window: positions below keep_first stay visible whatever the window has passed
#pragma once
#include "common.h"

struct AttnExtras {
  const float* sink;
  const float* rel;
  int rel_far;
  int keep_first;
};

// Whether the token at `pos` sees position p, for p <= pos.
__device__ __forceinline__ bool sees_position(int p, int pos, int window, int keep_first) {
  return p >= first_visible(pos, window) || p < keep_first;
}

__device__ __forceinline__ float distance_bias(const AttnExtras& x, int head, int distance) {
  return x.rel[(size_t)head * (x.rel_far + 1) + min(distance, x.rel_far)];
}

// The sink's share of a softmax whose running maximum is m (in the units of the scores) and whose sum is l:
// what has to be added to l.  A row that has seen nothing yet (m = -inf) is left to the caller.
__device__ __forceinline__ float sink_term(const AttnExtras& x, int head, float m) {
  return x.sink ? expf(x.sink[head] - m) : 0.f;
}
