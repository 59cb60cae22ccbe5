// Row-wise pieces of the online softmax, written for the transposed score layout (one lane = one
// query row, see cdna4.h).  These replace the warp-shuffle butterflies of the reference
// (reference: csrc/kernels/utils/reduce.h:16-100): here a row lives in 16*NT registers of two lanes, so a
// reduction is a register loop plus one exchange with lane^32.
#pragma once
#include "cdna4.h"

namespace aat {

// How far (log2 units) a row maximum may run ahead of the exponent's reference point before the
// running sum and output are rescaled.
constexpr float kLazyLog2 = 8.0f;

// max over the lane's registers of NT score tiles: one v_max3_f32 per two values, four chains.  Written as the
// instruction because hipcc re-associates fmaxf(m, fmaxf(a, b)) into two v_max_f32 and a v_max3_f32 per four
// values (48 instructions for 64 values instead of 34).
AAT_DEV float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
template <int NT> AAT_DEV float lane_max(const f16v (&s)[NT]) {
  float m[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) m[i] = fmaxf(s[0][2 * i], s[0][2 * i + 1]);
#pragma unroll
  for (int e = 8; e < NT * 16; e += 2) m[(e >> 1) & 3] = max3(m[(e >> 1) & 3], s[e >> 4][e & 15], s[e >> 4][(e & 15) + 1]);
  return max3(fmaxf(m[0], m[1]), m[2], m[3]);
}

// Set S^T entries above the causal diagonal to -inf.  kv_base = first kv index of score tile 0,
// q_lim = last kv index this lane's query row may see.  Register v of tile t holds kv index
// kv_base + 32 t + 4 h + (8 (v / 4) + v % 4): the lane-dependent part goes into one per-lane limit and every entry is
// then a comparison of that limit with a literal and a select -- no kv index per entry in a register, no branch.
AAT_DEV int causal_lane_limit(int kv_base, int q_lim, int h) { return q_lim - kv_base - 4 * h; }
template <int NT> AAT_DEV void causal_mask(f16v (&s)[NT], int kv_base, int q_lim, int h) {
  const int lim = causal_lane_limit(kv_base, q_lim, h);
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int v = 0; v < 16; ++v) s[t][v] = (32 * t + c_row(v, 0) > lim) ? -INFINITY : s[t][v];
  }
}

// Zero the P entries above the causal diagonal (same predicate as causal_mask).  exp2 of a masked
// score is already 0 for any positive scale; this pass makes the result exact for scale 0 as well,
// where -inf * 0 would otherwise leave a NaN.
template <int NT> AAT_DEV void zero_masked(f16v (&p)[NT], int kv_base, int q_lim, int h) {
  const int lim = causal_lane_limit(kv_base, q_lim, h);
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int v = 0; v < 16; ++v) p[t][v] = (32 * t + c_row(v, 0) > lim) ? 0.f : p[t][v];
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

// Lazy running max for one 32-row group: moves the exponent's reference point m_run and rescales
// l_run and the O accumulators only when some row of the wave has grown past it by more than
// kLazyLog2 in the log2 domain.  Until then P may exceed 1 by at most 2^kLazyLog2, which fp16 P and
// fp32 l, O absorb without loss; the final O / l is unchanged because numerator and denominator share
// the reference point.  Returns mc = m_run * c2, the term subtracted inside the exponent.
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

// s <- exp2(s*c2 - mc) in place (masked entries hold -inf and come out as 0 for any positive scale).
// FENCED: a scheduling barrier after every four entries, for kernels without a register to spare: left alone the
// scheduler lifts the multiply-adds of a whole tile above its exponentials and the results land in new registers.
template <int NT, bool FENCED = false> AAT_DEV void exp_tile(f16v (&s)[NT], float c2, float mc) {
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      s[t][v] = fast_exp2(__builtin_fmaf(s[t][v], c2, -mc));
      if constexpr (FENCED) {
        if (v % 4 == 3) __builtin_amdgcn_sched_barrier(0);
      }
    }
}

// exp of `count` consecutive entries (flattened index e = 16*tile + v) of a row group, in place.
// Used to spread the exponentials between the MFMAs of the next score tile.
template <int NT> AAT_DEV void exp_range(f16v (&s)[NT], int e0, int count, float c2, float mc) {
#pragma unroll
  for (int i = 0; i < count; ++i) {
    const int e = e0 + i;
    if (e < NT * 16) s[e >> 4][e & 15] = fast_exp2(__builtin_fmaf(s[e >> 4][e & 15], c2, -mc));
  }
}

// Round 16 kv rows (group g: score tile g/2, registers 8*(g%2) .. +7) of P to one fp16 MFMA operand and
// add their sum to `sum`.  The sum is taken in fp32 over the unrounded values with plain adds (two
// interleaved chains).  v_dot2_f32_f16 against a vector of ones would halve the instruction count, but on
// gfx950 the dot instructions share the matrix pipe's issue path: next to a wave that streams MFMAs each
// v_dot2c_f32_f16 of the other wave of the SIMD was measured at ~90 cycles instead of 4.5 (8 of them turned
// a 450-cycle stretch of exponentials and conversions into 1150 cycles), and a wave's own MFMAs wait for them too.
// PIN: the updated sum is tied to this point of the program.  Otherwise the compiler is free to sink the additions
// to the sum's next use -- the rescale test of the NEXT unit -- and the sixteen unrounded P values they read stay
// live across that unit's first contraction, which is where a kernel short of registers is shortest.
template <int NT, bool PIN = false> AAT_DEV void pack_p_group(h8 (&pf)[NT][2], const f16v (&s)[NT], int g, float& sum) {
  const int t = g >> 1, half = g & 1;
  h8 r;
  float s0 = s[t][8 * half] + s[t][8 * half + 1], s1 = s[t][8 * half + 2] + s[t][8 * half + 3];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const h2 pr = pack_rne(s[t][8 * half + 2 * i], s[t][8 * half + 2 * i + 1]);
    r[2 * i] = pr[0];
    r[2 * i + 1] = pr[1];
  }
  s0 += s[t][8 * half + 4] + s[t][8 * half + 5];
  s1 += s[t][8 * half + 6] + s[t][8 * half + 7];
  sum += s0 + s1;
  if constexpr (PIN) asm volatile("" : "+v"(sum));
  pf[t][half] = r;
}

}  // namespace aat
