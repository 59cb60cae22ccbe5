// Stand-alone benchmark of the RetNet parallel forward for MI355X: times hand-picked configurations of both
// kernels without Python and checks one (batch, head) slice of every result on the host (counterpart of
// reference benchmarks/retnet/retnet.cu:37-171 and its main :217-247; the recurrent form it also times has a
// benchmark of its own, retnet_recurrent.hip).
//
//   hipcc --offload-arch=gfx950 -O3 -fno-math-errno -ffp-contract=fast -fno-honor-nans \
//         -Xclang -target-feature -Xclang -packed-fp32-ops -I attention_autotuner_amd/csrc \
//         attention_autotuner_amd/csrc/benchmarks/retnet.hip -o retnet_bench
//   ./retnet_bench [B H Sq Sk] [--mask dense|causal|scan|decay] [--no-flush]
//
// d_qk = 256, d_v = 512 (RetNet's own head sizes).  q, k, v are N(0,1) fp16.  Every configuration is timed once
// per way of handing it the mask (see retnet_common.h); TFLOP/s counts 2*B*H*Sq*Sk*(d_qk+d_v) for the dense
// walk and the half of it on and below the diagonal for the other three.
#include "../kernels/retnet/regfuse/regfuse.h"
#include "../kernels/retnet/smemfuse/smemfuse.h"
#include "retnet_common.h"

using namespace retnet_bench;

constexpr int Kd = 256, D = 512;

struct Tensors {
  HostDevice<half_t> q, k, v, mask_dense, mask_decay, o;
  HostDevice<float> r, log2_gamma;
  void* scan = nullptr;
};

static MaskArgs mask_args(const Tensors& t, MaskKind m) {
  MaskArgs a;
  switch (m) {
    case MaskKind::Dense: a.mask = t.mask_dense.dev; a.walk_mode = aat::kMaskDense; break;
    case MaskKind::Causal: a.mask = t.mask_decay.dev; a.walk_mode = aat::kMaskCausal; break;
    case MaskKind::Scan: a.mask = t.mask_decay.dev; a.walk_mode = aat::kMaskScan; a.workspace = t.scan; break;
    case MaskKind::Decay: a.log2_gamma = t.log2_gamma.dev; break;
  }
  return a;
}

// o and r of slice (B-1, H-1) in `rows` query rows against S = (q k^T) * mask, r = max(sum |S|, 1), o = (S / r) v.
static Agreement check_slice(const ProblemShape& ps, Tensors& t, MaskKind m) {
  t.o.download();
  t.r.download();
  const int bh = ps.B * ps.H - 1, h = ps.H - 1;
  const float gamma = gammas(ps.H)[h];
  const half_t* q = t.q.host.data() + (size_t)bh * ps.Sq * Kd;
  const half_t* k = t.k.host.data() + (size_t)bh * ps.Sk * Kd;
  const half_t* v = t.v.host.data() + (size_t)bh * ps.Sk * D;
  const half_t* mask = (m == MaskKind::Dense ? t.mask_dense : t.mask_decay).host.data() + (size_t)h * ps.Sq * ps.Sk;
  Agreement a;
  std::vector<double> s(ps.Sk), out(D);
  const int n_rows = 48;
  for (int n = 0; n < n_rows; ++n) {
    const int i = (int)((long)n * (ps.Sq - 1) / (n_rows - 1));
    double rsum = 0;
    for (int j = 0; j < ps.Sk; ++j) {
      const double mk = m == MaskKind::Decay ? decay_value(gamma, i + ps.Sk - ps.Sq - j) : (double)(float)mask[(size_t)i * ps.Sk + j];
      double acc = 0;
      if (mk != 0.0)
        for (int c = 0; c < Kd; ++c) acc += (double)(float)q[(size_t)i * Kd + c] * (double)(float)k[(size_t)j * Kd + c];
      s[j] = acc * mk;
      rsum += std::fabs(s[j]);
    }
    const double r = std::max(rsum, 1.0);
    std::fill(out.begin(), out.end(), 0.0);
    for (int j = 0; j < ps.Sk; ++j) {
      if (s[j] == 0.0) continue;
      const double p = s[j] / r;
      for (int c = 0; c < D; ++c) out[c] += p * (double)(float)v[(size_t)j * D + c];
    }
    for (int c = 0; c < D; ++c) a.add((double)(float)t.o.host[((size_t)bh * ps.Sq + i) * D + c], out[c]);
    const double got_r = t.r.host[(size_t)bh * ps.Sq + i];
    a.bad += !(std::fabs(got_r - r) <= 2e-3 * r);      // r is fp32 on the GPU: sums of fp32 products in another order
  }
  return a;
}

static void report(const char* what, const ProblemShape& ps, MaskKind m, const aat_bench::Timing& t, const Agreement& a) {
  const double fl = 2.0 * ps.B * ps.H * (double)ps.Sq * ps.Sk * (Kd + D) * share_of_dense(m);
  std::printf("%-58s mask %-6s mean %.4f ms  median %.4f  p20 %.4f  p80 %.4f  (%d launches)  %.1f TFLOP/s = %.1f%% of 2.5 PFLOP/s"
              "  check: max |err| %.2e of %.2f -> %s\n", what, name_of(m), t.mean_ms, t.median_ms, t.p20_ms, t.p80_ms, t.launches,
              fl / t.median_ms * 1e-9, fl / t.median_ms * 1e-9 / 25.0, a.max_err, a.max_ref, a.ok() ? "ok" : "MISMATCH");
}

static int g_failures = 0;

template <class Plain, class Decay>
static void run_all_masks(const char* what, const ProblemShape& ps, Tensors& t, int Br, int Bc, int threads, int lds_bytes,
                          Plain plain, Decay decay) {
  if (ps.Sq % Br || ps.Sk % Bc) {
    std::printf("%-58s skipped: Sq %% %d or Sk %% %d\n", what, Br, Bc);
    return;
  }
  HIP_OK(hipFuncSetAttribute((const void*)plain, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
  HIP_OK(hipFuncSetAttribute((const void*)decay, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
  const dim3 grid(ps.B * ps.H * (ps.Sq / Br)), block(threads);
  for (MaskKind m : kAllMasks) {
    if (ps.only && std::strcmp(ps.only, name_of(m))) continue;
    const MaskArgs a = mask_args(t, m);
    auto launch = [&] {
      if (m == MaskKind::Decay) {
        decay<<<grid, block, lds_bytes, 0>>>(t.q.dev, t.k.dev, t.v.dev, nullptr, t.o.dev, t.r.dev, ps.H, ps.Sk, ps.Sq, 1, a.log2_gamma, nullptr);
        return;
      }
      aat::MaskWalk walk;
      HIP_OK(aat::prepare_mask_walk(a.walk_mode, a.mask, ps.H, ps.Sq, ps.Sk, a.workspace, 0, &walk));
      plain<<<grid, block, lds_bytes, 0>>>(t.q.dev, t.k.dev, t.v.dev, a.mask, t.o.dev, t.r.dev, ps.H, ps.Sk, ps.Sq, walk.causal, nullptr,
                                           walk.extents);
    };
    HIP_OK(hipMemset(t.o.dev, 0xff, t.o.host.size() * sizeof(half_t)));
    launch();
    HIP_OK(hipDeviceSynchronize());
    const Agreement agree = check_slice(ps, t, m);
    g_failures += !agree.ok();
    report(what, ps, m, aat_bench::do_bench(launch, ps.flush), agree);
  }
}

// Register-fused: <Br, Bc, threads, K buffers, V buffers, mask buffers, waves per SIMD>
template <int Br, int Bc, int NT, int NSK, int NSV, int NSM, int WPE>
static void test_regfuse_retnet(const ProblemShape& ps, Tensors& t) {
  using T = aat::RetFwdRegfuse<Kd, D, Br, Bc, NT, NSK, NSV, NSM>;
  char name[128];
  std::snprintf(name, sizeof name, "regfuse  Br=%d Bc=%d thr=%d bufs=%d/%d/%d waves/SIMD=%d", Br, Bc, NT, NSK, NSV, NSM, WPE);
  run_all_masks(name, ps, t, Br, Bc, NT, T::kSmemBytes, &aat::ret_fwd_regfuse<Kd, D, Br, Bc, NT, NSK, NSV, NSM, WPE, false>,
                &aat::ret_fwd_regfuse<Kd, D, Br, Bc, NT, NSK, NSV, NSM, WPE, true>);
}

// LDS-fused: <Br, Bc, threads, K buffers, V buffers, mask buffers, waves along kv, waves along d, waves per SIMD>
template <int Br, int Bc, int NT, int NSK, int NSV, int NSM, int W1N, int W2N, int WPE>
static void test_smemfuse_retnet(const ProblemShape& ps, Tensors& t) {
  using T = aat::RetFwdSmemfuse<Kd, D, Br, Bc, NT, NSK, NSV, NSM, W1N, W2N>;
  char name[128];
  std::snprintf(name, sizeof name, "smemfuse Br=%d Bc=%d thr=%d bufs=%d/%d/%d grid=%dx%d waves/SIMD=%d", Br, Bc, NT, NSK, NSV, NSM, W1N, W2N, WPE);
  run_all_masks(name, ps, t, Br, Bc, NT, T::kSmemBytes, &aat::ret_fwd_smemfuse<Kd, D, Br, Bc, NT, NSK, NSV, NSM, W1N, W2N, WPE, false>,
                &aat::ret_fwd_smemfuse<Kd, D, Br, Bc, NT, NSK, NSV, NSM, W1N, W2N, WPE, true>);
}

int main(int argc, char** argv) {
  ProblemShape ps;
  if (!parse_args(argc, argv, &ps)) {
    std::printf("usage: %s [B H Sq Sk] [--mask dense|causal|scan|decay] [--no-flush]\n", argv[0]);
    return 2;
  }
  hipDeviceProp_t prop;
  HIP_OK(hipGetDeviceProperties(&prop, 0));
  std::printf("%s  %d CUs  LDS/block %zu KB   RetNet forward B=%d H=%d Sq=%d Sk=%d d_qk=%d d_v=%d fp16 %s\n", prop.gcnArchName,
              prop.multiProcessorCount, prop.sharedMemPerBlockOptin / 1024, ps.B, ps.H, ps.Sq, ps.Sk, Kd, D,
              ps.flush ? "(cache flushed before every launch)" : "(hot cache)");
  Tensors t;
  t.q = randn((size_t)ps.B * ps.H * ps.Sq * Kd, 1);
  t.k = randn((size_t)ps.B * ps.H * ps.Sk * Kd, 2);
  t.v = randn((size_t)ps.B * ps.H * ps.Sk * D, 3);
  t.mask_dense = randn((size_t)ps.H * ps.Sq * ps.Sk, 4);
  t.mask_decay = decay_mask(ps.H, ps.Sq, ps.Sk);
  t.log2_gamma = log2_gammas(ps.H);
  t.o = empty<half_t>((size_t)ps.B * ps.H * ps.Sq * D);
  t.r = empty<float>((size_t)ps.B * ps.H * ps.Sq);
  HIP_OK(hipMalloc(&t.scan, aat::mask_extent_bytes(ps.H, ps.Sq, ps.Sk)));

  test_smemfuse_retnet<128, 64, 512, 1, 1, 1, 2, 8, 2>(ps, t);
  test_smemfuse_retnet<128, 64, 512, 1, 1, 1, 2, 4, 2>(ps, t);
  test_smemfuse_retnet<64, 64, 256, 1, 1, 1, 2, 4, 1>(ps, t);
  test_regfuse_retnet<128, 32, 256, 1, 1, 1, 1>(ps, t);
  test_regfuse_retnet<128, 64, 256, 1, 1, 1, 1>(ps, t);

  for (auto* x : {&t.q, &t.k, &t.v, &t.mask_dense, &t.mask_decay, &t.o}) x->release();
  t.r.release();
  t.log2_gamma.release();
  HIP_OK(hipFree(t.scan));
  if (g_failures) std::printf("%d result(s) disagree with the host formulas\n", g_failures);
  return g_failures ? 1 : 0;
}
