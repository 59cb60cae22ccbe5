// Row-wise pieces of the online softmax and of the RetNet abs-sum normalisation, written for the
// transposed score layout (one lane = one query row, see cdna4.h).  These replace the warp-shuffle
// butterflies of the reference (reference: csrc/kernels/utils/reduce.h:16-100, elementwise.h:5-41):
// here a row lives in 16*NT registers of two lanes, so a reduction is a register loop plus one
// exchange with lane^32.
#pragma once
#include "cdna4.h"

namespace aat {

// max over the lane's registers of NT score tiles
template <int NT> AAT_DEV float lane_max(const f16v (&s)[NT]) {
  float m = -INFINITY;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int v = 0; v < 16; v += 2) m = fmaxf(m, fmaxf(s[t][v], s[t][v + 1]));  // v_max3_f32
  }
  return m;
}

// Set S^T entries above the causal diagonal to -inf.  kv_base = first kv index of score tile 0,
// q_lim = last kv index this lane's query row may see.
template <int NT> AAT_DEV void causal_mask(f16v (&s)[NT], int kv_base, int q_lim, int h) {
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int kv = kv_base + 32 * t + c_row(v, h);
      if (kv > q_lim) s[t][v] = -INFINITY;
    }
  }
}

}  // namespace aat
