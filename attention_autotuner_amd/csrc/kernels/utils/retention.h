// Row-wise pieces of RetNet's abs-sum normalisation, for the transposed score layout (cdna4.h).
// Replaces multiply_mask / update_r of the reference (reference: csrc/kernels/utils/elementwise.h:5-41) and
// reduce_sumabs (reference: csrc/kernels/utils/reduce.h:3-14).
//
// The reference keeps O normalised at every step: r_new = max(R, 1) with R the running sum of |S|,
// O = O * r_old / r_new + half(S / r_new) V.  Here the normaliser is lazy: P = S / r_ref with a
// reference r_ref that moves only when R outgrows it by kLazyRatio, and the exact max(R, 1) is applied
// once in the epilogue (O *= r_ref / max(R, 1)).  |P| <= kLazyRatio, which fp16 holds with the same
// relative precision as values below 1; the result differs from the reference's only in which
// power-of-two-ish scale the fp16 rounding of P happens at.
#pragma once
#include "cdna4.h"

namespace aat {

constexpr float kLazyRatio = 256.0f;

struct RetentionRow {
  float big_r;   // running sum of |S| over the kv range seen so far (whole row: both lanes hold it)
  float r_ref;   // scale P is currently divided by (>= 1)
};

// S <- S * mask for one 32-row group of a Bc-wide tile.  maddr[4*t + g] is the LDS address of this
// lane's four mask values for score tile t, registers 4g .. 4g+3 (kv rows 8g + 4h + 0..3 of the tile).
template <int NT>
AAT_DEV void apply_mask(f16v (&s)[NT], const uint32_t (&maddr)[NT * 4], int buf_off) {
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const h4 m = *reinterpret_cast<AAT_AS3 const h4*>((uintptr_t)(maddr[4 * t + g] + buf_off));
#pragma unroll
      for (int e = 0; e < 4; ++e) s[t][4 * g + e] *= (float)m[e];
    }
  }
}

// Fold one masked score tile into the row statistics and turn it into P = S / r_ref (in place).
// Rescales the O accumulators when the reference scale moves.
// ACC_PIN: the O accumulators live in accumulation registers (kernels above 256 registers); rescale
// them one 16-register block at a time so the copies through vector registers stay short-lived.
template <int NT, int DT, bool ACC_PIN = false>
AAT_DEV void retention_step(f16v (&s)[NT], RetentionRow& row, f16v (&oacc)[DT]) {
  float part = 0.f;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) part += __builtin_fabsf(s[t][v]);
  row.big_r += pair_sum(part);
  const bool grow = row.big_r > kLazyRatio * row.r_ref;
  if (__builtin_amdgcn_ballot_w64(grow) != 0) {                     // wave-uniform branch
    const float r_new = fmaxf(row.big_r, 1.0f);
    const float alpha = row.r_ref * fast_rcp(r_new);
    row.r_ref = r_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[dt][v] *= alpha;
      if constexpr (ACC_PIN) asm volatile("" : "+a"(oacc[dt]));
    }
  }
  const float inv = fast_rcp(row.r_ref);
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) s[t][v] *= inv;
}

// Round 16 kv rows of P to one fp16 MFMA operand (no sum needed here).
template <int NT> AAT_DEV void pack_group(h8 (&pf)[NT][2], const f16v (&s)[NT], int g) {
  pf[g >> 1][g & 1] = pack8_rne(s[g >> 1], 8 * (g & 1));
}

}  // namespace aat
