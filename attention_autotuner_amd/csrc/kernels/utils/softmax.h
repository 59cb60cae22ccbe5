// Row-wise pieces of the online softmax and of the RetNet abs-sum normalisation, written for the
// transposed score layout (one lane = one query row, see cdna4.h).  These replace the warp-shuffle
// butterflies of the reference (reference: csrc/kernels/utils/reduce.h:16-100, elementwise.h:5-41):
// here a row lives in 16*NT registers of two lanes, so a reduction is a register loop plus one
// exchange with lane^32.
#pragma once
#include "cdna4.h"

namespace aat {

// How far (log2 units) a row maximum may run ahead of the exponent's reference point before the
// running sum and output are rescaled.
constexpr float kLazyLog2 = 8.0f;

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

// One step of the running-max recurrence.  m_old / m_new are UNSCALED row maxima (-inf before the
// first visible kv), c2 = softmax_scale * log2(e).  alpha rescales the running sum and output,
// mc is the term subtracted inside the exponent.  Written so that -inf never meets a multiply:
// a row that has seen nothing yet keeps alpha = 1 (its l and O are still zero).
struct SoftmaxStep {
  float alpha, mc;
};
AAT_DEV SoftmaxStep softmax_step(float m_old, float m_new, float c2) {
  const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
  const float m_prev = (m_old == -INFINITY) ? m_use : m_old;
  SoftmaxStep st;
  st.alpha = fast_exp2((m_prev - m_use) * c2);
  st.mc = m_use * c2;
  return st;
}

// s <- exp2(s*c2 - mc) in place; returns the lane's partial row sum.  MASKED zeroes the entries above
// the causal diagonal explicitly (exact for any scale, including 0) and is used on diagonal tiles only.
template <int NT, bool MASKED>
AAT_DEV float exp_tile(f16v (&s)[NT], float c2, float mc, int kv_base, int q_lim, int h) {
  float lsum = 0.f;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      float p;
      if (MASKED && kv_base + 32 * t + c_row(v, h) > q_lim) p = 0.f;
      else p = fast_exp2(__builtin_fmaf(MASKED ? fmaxf(s[t][v], -3.0e38f) : s[t][v], c2, -mc));
      s[t][v] = p;
      lsum += p;
    }
  }
  return lsum;
}

}  // namespace aat
