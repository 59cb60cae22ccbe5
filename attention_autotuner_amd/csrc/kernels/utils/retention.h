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

// The same from one address register.  In a Rows16-swizzled tile whose rows are a power of two of chunks, chunk i
// of a row sits at (row start + 16 (i ^ x)) with x fixed per row; a row starts at a multiple of its own size (the
// buffer does too), so that is (address of the row's chunk 0) ^ 16 i.  chunk0 = that address + 8h.
template <int NT>
AAT_DEV void apply_mask_folded(f16v (&s)[NT], uint32_t chunk0, int buf_off) {
  asm volatile("" : "+v"(chunk0));      // or the 4 NT addresses are computed once, ahead of the loop, and kept in registers
#pragma unroll
  for (int t = 0; t < NT; ++t) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const h4 m = *reinterpret_cast<AAT_AS3 const h4*>((uintptr_t)((chunk0 ^ (uint32_t)((4 * t + g) << 4)) + buf_off));
#pragma unroll
      for (int e = 0; e < 4; ++e) s[t][4 * g + e] *= (float)m[e];
    }
  }
}

// apply_mask_folded with the reads issued behind the compiler's back.  In front of an LDS read it can see, the compiler
// waits for every LDS-DMA copy in flight (it takes them for writes the read may depend on): the copy of the next tile,
// threaded between the matrix steps before this point, would be waited for here.
template <int NT>
AAT_DEV void apply_mask_folded_blind(f16v (&s)[NT], uint32_t chunk0) {
  h4 m[NT * 4];
#pragma unroll
  for (int i = 0; i < NT * 4; ++i) {
    const uint32_t a = chunk0 ^ (uint32_t)(i << 4);
    asm volatile("ds_read_b64 %0, %1" : "=v"(m[i]) : "v"(a));
  }
  asm volatile("s_waitcnt lgkmcnt(0)");
#pragma unroll
  for (int i = 0; i < NT * 4; ++i) asm volatile("" : "+v"(m[i]));       // no use of m[i] above the wait
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) s[t][4 * g + e] *= (float)m[4 * t + g][e];
}

// Decay mask evaluated in registers instead of read from a [H, S_q, S_kv] tensor.  The reference always
// streams the tensor (reference: python/ops/retnet_interface.py:26-31) and lists "causal config" and the
// mask stream's cost ("retnet performance issue ... mask stage 2?") as open items (README.md:102-114):
//     D[q][kv] = gamma^(q + diag - kv)  for kv <= q + diag,   0 above the diagonal,   diag = S_kv - S_q.
// In the transposed score layout a lane owns one index and its 16*NT registers run over the other one
// at fixed offsets off(t, v) = 32t + 8(v/4) + 4h + v%4 from the tile origin, so with lg = log2(gamma)
//     D = exp2(lg * base) * fac(t, v)
// is one per-lane scalar per tile times per-lane constants:
//     OWN_Q  (lane owns q, registers run over kv):  base = (q + diag) - kv_origin,  fac = exp2(-lg * off)
//     !OWN_Q (lane owns kv, registers run over q):  base = q_origin - (kv - diag),  fac = exp2(+lg * off)
// Off the diagonal |lg| * tile_rows bounds the exponents, so nothing overflows for gamma >= 0.5 and
// tiles of up to 128 rows; far below the diagonal the scalar underflows to zero, as the fp16 tensor does.
// The offsets split as off = (32t + 8g) + (4h + e) with v = 4g + e, so the 16*NT constants are products
// of 4*NT + 4 of them: fb[t][g] = exp2(-/+lg * (32t + 8g)), fa[e] = exp2(-/+lg * e), all of them the same in
// every lane, with the half-wave's share exp2(-/+lg * 4h) folded into the per-tile scalar.
template <int NT, bool OWN_Q>
struct DecayMask {
  float fa[4], fb[NT][4];
  float lg;
  int h4;

  // The rate belongs to the head, so lg and the 4*NT factors fb are the same in every lane: passed through
  // readfirstlane they live in scalar registers (a two-wave kernel at the 256-register limit has none to spare).
  AAT_DEV static float uniform(float x) { return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(x))); }
  AAT_DEV void init(float lg2gamma, int h) {
    lg = uniform(lg2gamma);
    h4 = 4 * h;
    const float step = OWN_Q ? -lg : lg;
#pragma unroll
    for (int e = 0; e < 4; ++e) fa[e] = uniform(fast_exp2(step * (float)e));   // the half-wave's 4h goes into the tile scalar
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) fb[t][g] = uniform(fast_exp2(step * (float)(32 * t + 8 * g)));
  }
  // s <- s * D * extra for the tile whose origin makes `base` (see above).  DIAG: the diagonal may cross
  // this tile, entries above it are zeroed.
  template <bool DIAG, class Extra>
  AAT_DEV void apply(f16v (&s)[NT], int base, Extra&& extra) const {
    const int own = OWN_Q ? base - h4 : base + h4;        // this lane's distance to the diagonal at register 0
    const float tf = fast_exp2(lg * (float)own);
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float tg = tf * fb[t][g];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int v = 4 * g + e;
          float m = tg * fa[e] * extra(t, v);
          if constexpr (DIAG) {          // against a literal: base -/+ (offset + 4h) per register would be 16 NT values kept per lane
            const int off = 32 * t + 8 * g + e;
            if ((OWN_Q ? own - off : own + off) < 0) m = 0.f;
          }
          s[t][v] *= m;
        }
      }
  }
};

// O <- O * alpha for one 32-row group.  IN_PLACE: the accumulators live in accumulation registers (kernels above 256
// registers) and are multiplied there, one register at a time, by hand: given the loop the compiler reads dozens of
// accumulation registers ahead of the multiplications and spills vector registers to make room for them.  The matrix
// instructions that last wrote these registers are a whole score contraction back, so no read here needs a wait.
template <int DT, bool IN_PLACE>
AAT_DEV void rescale_acc(f16v (&oacc)[DT], float alpha) {
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      if constexpr (IN_PLACE) {
        float x = oacc[dt][v], t;
        asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %2, %1\n\tv_accvgpr_write_b32 %0, %1"
                     : "+a"(x), "=&v"(t) : "v"(alpha));
        oacc[dt][v] = x;
      } else {
        oacc[dt][v] *= alpha;
      }
    }
  // The compiler does not see the writes above and inserts no wait states between the last of them and a matrix
  // instruction that takes the register as its addend; this runs once in hundreds of tiles.
  if constexpr (IN_PLACE) asm volatile("s_nop 3" : "+a"(oacc[DT - 1]));
}

// Fold one masked score tile into the row statistics and turn it into P = S / r_ref (in place).
// Rescales the O accumulators when the reference scale moves.
// ACC_PIN: the O accumulators live in accumulation registers (kernels above 256 registers) and are rescaled there.
// rescale(alpha): multiplies the row group's O accumulators, wherever they live.
template <int NT, class Rescale>
AAT_DEV void retention_step_with(f16v (&s)[NT], RetentionRow& row, Rescale&& rescale) {
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
    rescale(alpha);
  }
  const float inv = fast_rcp(row.r_ref);
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) s[t][v] *= inv;
}
template <int NT, int DT, bool ACC_PIN = false>
AAT_DEV void retention_step(f16v (&s)[NT], RetentionRow& row, f16v (&oacc)[DT]) {
  retention_step_with<NT>(s, row, [&](float alpha) { rescale_acc<DT, ACC_PIN>(oacc, alpha); });
}

// Round 16 kv rows of P to one fp16 MFMA operand (no sum needed here).
template <int NT> AAT_DEV void pack_group(h8 (&pf)[NT][2], const f16v (&s)[NT], int g) {
  pf[g >> 1][g & 1] = pack8_rne(s[g >> 1], 8 * (g & 1));
}

}  // namespace aat
