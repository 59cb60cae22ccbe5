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

namespace aat {

// Lazy running max for one 32-row group (see kLazyLog2): moves the exponent's reference point m_run
// and rescales l_run and the O accumulators only when some row of the wave outgrew it.  Returns
// mc = m_run * c2, the term subtracted inside the exponent for this tile.
template <int NT, int DT>
AAT_DEV float lazy_max_step(const f16v (&s)[NT], float& m_run, float& l_run, f16v (&oacc)[DT], float c2) {
  const float m_tile = pair_max(lane_max<NT>(s));
  const bool grow = (m_tile - m_run) * c2 > kLazyLog2;             // false for -inf - -inf
  if (__builtin_amdgcn_ballot_w64(grow) != 0) {                     // wave-uniform branch
    const float m_new = fmaxf(m_run, m_tile);
    const SoftmaxStep st = softmax_step(m_run, m_new, c2);
    m_run = m_new;
    l_run *= st.alpha;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[dt][v] *= st.alpha;
  }
  return (m_run == -INFINITY ? 0.f : m_run) * c2;
}

// exp of `count` consecutive entries (flattened index e = 16*tile + v) of a row group, in place;
// returns their sum.  Used to spread the exponentials between the MFMAs of the next score tile.
template <int NT, bool MASKED>
AAT_DEV float exp_range(f16v (&s)[NT], int e0, int count, float c2, float mc, int kv_base, int q_lim, int h) {
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < count; ++i) {
    const int e = e0 + i;
    if (e < NT * 16) {
      const int t = e >> 4, v = e & 15;
      float p;
      if (MASKED && kv_base + 32 * t + c_row(v, h) > q_lim) p = 0.f;
      else p = fast_exp2(__builtin_fmaf(MASKED ? fmaxf(s[t][v], -3.0e38f) : s[t][v], c2, -mc));
      s[t][v] = p;
      sum += p;
    }
  }
  return sum;
}

template <int NT> AAT_DEV void pack_p(h8 (&pf)[NT][2], const f16v (&s)[NT]) {
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    pf[t][0] = pack8_rne(s[t], 0);
    pf[t][1] = pack8_rne(s[t], 8);
  }
}

}  // namespace aat
