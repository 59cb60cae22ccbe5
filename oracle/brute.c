/* fp64 brute-force loops for attention forward, RetNet forward, RetNet backward and the RetNet recurrent form.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is an independent restatement (plain loops, double
 * precision, no tiling, no library calls besides exp) used to pin oracle/ref_op.py, which in turn
 * checks the HIP kernels.  Formulas: reference python/utils/ref_op.py:2-13 and, for the gradients,
 * reference csrc/kernels/retnet/bwd/bwd_colblock.h:522-576; the recurrent form restates the scan of
 * reference csrc/kernels/retnet/recurrent/recurrent.h:110-114 (the pair operator) and :303-330 (one scan per
 * (key dim, value dim) pair, seeded with (0, 0), its .y component weighted by q and summed over key dims).
 *
 * All tensors are contiguous fp32: q [BH,Sq,Kd], k [BH,Sk,Kd], v [BH,Sk,D], mask [H,Sq,Sk] (the
 * head of slice b is b % H), outputs likewise.  Built by oracle/Makefile into oracle/libbrute.so.
 */
#include <math.h>
#include <stdlib.h>

void brute_attention_fwd(const float* q, const float* k, const float* v, float* o, int BH, int Sq,
                         int Sk, int Kd, int D, double scale, int causal) {
  double* p = (double*)malloc(sizeof(double) * (size_t)Sk);
  for (int b = 0; b < BH; ++b)
    for (int i = 0; i < Sq; ++i) {
      const int lim = causal ? i + (Sk - Sq) : Sk - 1;
      double mx = -HUGE_VAL;
      for (int j = 0; j <= lim && j < Sk; ++j) {
        double acc = 0;
        for (int c = 0; c < Kd; ++c)
          acc += (double)q[((size_t)b * Sq + i) * Kd + c] * (double)k[((size_t)b * Sk + j) * Kd + c];
        p[j] = acc * scale;
        if (p[j] > mx) mx = p[j];
      }
      double l = 0;
      for (int j = 0; j <= lim && j < Sk; ++j) { p[j] = exp(p[j] - mx); l += p[j]; }
      for (int d = 0; d < D; ++d) {
        double acc = 0;
        for (int j = 0; j <= lim && j < Sk; ++j) acc += p[j] * (double)v[((size_t)b * Sk + j) * D + d];
        o[((size_t)b * Sq + i) * D + d] = l > 0 ? (float)(acc / l) : 0.f;
      }
    }
  free(p);
}

void brute_retnet_fwd(const float* q, const float* k, const float* v, const float* mask, float* o,
                      float* r, int BH, int H, int Sq, int Sk, int Kd, int D) {
  double* s = (double*)malloc(sizeof(double) * (size_t)Sk);
  for (int b = 0; b < BH; ++b)
    for (int i = 0; i < Sq; ++i) {
      double R = 0;
      for (int j = 0; j < Sk; ++j) {
        double acc = 0;
        for (int c = 0; c < Kd; ++c)
          acc += (double)q[((size_t)b * Sq + i) * Kd + c] * (double)k[((size_t)b * Sk + j) * Kd + c];
        s[j] = acc * (double)mask[((size_t)(b % H) * Sq + i) * Sk + j];
        R += fabs(s[j]);
      }
      if (R < 1.0) R = 1.0;
      r[(size_t)b * Sq + i] = (float)R;
      for (int d = 0; d < D; ++d) {
        double acc = 0;
        for (int j = 0; j < Sk; ++j) acc += s[j] * (double)v[((size_t)b * Sk + j) * D + d];
        o[((size_t)b * Sq + i) * D + d] = (float)(acc / R);
      }
    }
  free(s);
}

/* Gradients with r held constant (the reference detaches it). */
void brute_retnet_bwd(const float* q, const float* k, const float* v, const float* mask,
                      const float* dout, float* dq, float* dk, float* dv, int BH, int H, int Sq,
                      int Sk, int Kd, int D) {
  double* P = (double*)malloc(sizeof(double) * (size_t)Sq * Sk);
  double* dS = (double*)malloc(sizeof(double) * (size_t)Sq * Sk);
  for (int b = 0; b < BH; ++b) {
    const float* qb = q + (size_t)b * Sq * Kd;
    const float* kb = k + (size_t)b * Sk * Kd;
    const float* vb = v + (size_t)b * Sk * D;
    const float* gb = dout + (size_t)b * Sq * D;
    const float* mb = mask + (size_t)(b % H) * Sq * Sk;
    for (int i = 0; i < Sq; ++i) {
      double R = 0;
      for (int j = 0; j < Sk; ++j) {
        double acc = 0;
        for (int c = 0; c < Kd; ++c) acc += (double)qb[(size_t)i * Kd + c] * (double)kb[(size_t)j * Kd + c];
        P[(size_t)i * Sk + j] = acc * (double)mb[(size_t)i * Sk + j];
        R += fabs(P[(size_t)i * Sk + j]);
      }
      if (R < 1.0) R = 1.0;
      for (int j = 0; j < Sk; ++j) {
        P[(size_t)i * Sk + j] /= R;
        double acc = 0;
        for (int d = 0; d < D; ++d) acc += (double)gb[(size_t)i * D + d] * (double)vb[(size_t)j * D + d];
        dS[(size_t)i * Sk + j] = acc / R * (double)mb[(size_t)i * Sk + j];
      }
    }
    for (int j = 0; j < Sk; ++j) {
      for (int d = 0; d < D; ++d) {
        double acc = 0;
        for (int i = 0; i < Sq; ++i) acc += P[(size_t)i * Sk + j] * (double)gb[(size_t)i * D + d];
        dv[((size_t)b * Sk + j) * D + d] = (float)acc;
      }
      for (int c = 0; c < Kd; ++c) {
        double acc = 0;
        for (int i = 0; i < Sq; ++i) acc += dS[(size_t)i * Sk + j] * (double)qb[(size_t)i * Kd + c];
        dk[((size_t)b * Sk + j) * Kd + c] = (float)acc;
      }
    }
    for (int i = 0; i < Sq; ++i)
      for (int c = 0; c < Kd; ++c) {
        double acc = 0;
        for (int j = 0; j < Sk; ++j) acc += dS[(size_t)i * Sk + j] * (double)kb[(size_t)j * Kd + c];
        dq[((size_t)b * Sq + i) * Kd + c] = (float)acc;
      }
  }
  free(P);
  free(dS);
}

/* RetNet recurrent form.  q, k [BH][kdim][L], v, out [BH][vdim][L] (sequence contiguous), decay [H][L]:
 *   S(kd, vd, n) = decay[n] * S(kd, vd, n-1) + k[kd][n] * v[vd][n],  S(., ., -1) = 0
 *   out[vd][n]   = sum_{kd < block_kdim} q[kd][n] * S(kd, vd, n) */
void brute_retnet_recurrent(const float* q, const float* k, const float* v, const float* decay, float* out,
                            int BH, int H, int kdim, int vdim, int L, int block_kdim) {
  double* acc = (double*)malloc(sizeof(double) * (size_t)L);
  for (int b = 0; b < BH; ++b) {
    const float* a = decay + (size_t)(b % H) * L;
    for (int vd = 0; vd < vdim; ++vd) {
      const float* vr = v + ((size_t)b * vdim + vd) * L;
      for (int n = 0; n < L; ++n) acc[n] = 0;
      for (int kd = 0; kd < block_kdim; ++kd) {
        const float* kr = k + ((size_t)b * kdim + kd) * L;
        const float* qr = q + ((size_t)b * kdim + kd) * L;
        double S = 0;
        for (int n = 0; n < L; ++n) {
          S = (double)a[n] * S + (double)kr[n] * (double)vr[n];
          acc[n] += (double)qr[n] * S;
        }
      }
      for (int n = 0; n < L; ++n) out[((size_t)b * vdim + vd) * L + n] = (float)acc[n];
    }
  }
  free(acc);
}
