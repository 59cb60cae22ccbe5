// Stand-alone benchmark of the RetNet parallel backward for MI355X: times hand-picked configurations of the three
// chained-contraction passes (dV, dK, dQ) without Python and checks rows of one (batch, head) slice of every
// gradient on the host (counterpart of reference benchmarks/retnet/retnet_bwd.cu:36-147 and its main :184-211).
//
//   hipcc --offload-arch=gfx950 -O3 -fno-math-errno -ffp-contract=fast -fno-honor-nans \
//         -Xclang -target-feature -Xclang -packed-fp32-ops -I attention_autotuner_amd/csrc \
//         attention_autotuner_amd/csrc/benchmarks/retnet_bwd.hip -o retnet_bwd_bench
//   ./retnet_bwd_bench [B H Sq Sk] [--mask dense|causal|scan|decay] [--no-flush]
//
// d_qk = 256, d_v = 512.  q, k, v, dO are N(0,1) fp16; r comes from the forward kernel, as it does in training.
// One timed launch = the three passes (for `scan` the ranges are those the forward's scan left behind, as in the
// operator).  TFLOP/s counts the five contractions, 2*B*H*Sq*Sk*(3 d_qk + 2 d_v), halved for the walks that
// skip the tiles above the diagonal.
#include "../kernels/retnet/bwd/bwd_chain.h"
#include "../kernels/retnet/bwd/dk_from_ds.h"
#include "../kernels/retnet/smemfuse/smemfuse.h"
#include "retnet_common.h"

using namespace retnet_bench;
using aat::BwdPass;

constexpr int Kd = 256, D = 512;

struct Tensors {
  HostDevice<half_t> q, k, v, dout, mask_dense, mask_decay, o, dq, dk, dv;
  HostDevice<float> r, log2_gamma;
  void* scan = nullptr;
  half_t* ds = nullptr;          // [B*H, Sq, Sk]: dS as the row pass forms it, for the dK kernel that reads it back
};

// r (and the scan of the decay mask) as the forward leaves them.
static void forward_for(const ProblemShape& ps, Tensors& t, MaskKind m) {
  constexpr int Br = 128, Bc = 64, NT = 512;
  using T = aat::RetFwdSmemfuse<Kd, D, Br, Bc, NT, 1, 1, 1, 2, 8>;
  auto plain = &aat::ret_fwd_smemfuse<Kd, D, Br, Bc, NT, 1, 1, 1, 2, 8, 2, false>;
  auto decay = &aat::ret_fwd_smemfuse<Kd, D, Br, Bc, NT, 1, 1, 1, 2, 8, 2, true>;
  HIP_OK(hipFuncSetAttribute((const void*)plain, hipFuncAttributeMaxDynamicSharedMemorySize, T::kSmemBytes));
  HIP_OK(hipFuncSetAttribute((const void*)decay, hipFuncAttributeMaxDynamicSharedMemorySize, T::kSmemBytes));
  const dim3 grid(ps.B * ps.H * (ps.Sq / Br)), block(NT);
  if (m == MaskKind::Decay) {
    decay<<<grid, block, T::kSmemBytes, 0>>>(t.q.dev, t.k.dev, t.v.dev, nullptr, t.o.dev, t.r.dev, ps.H, ps.Sk, ps.Sq, 1, t.log2_gamma.dev, nullptr);
  } else {
    const half_t* mask = m == MaskKind::Dense ? t.mask_dense.dev : t.mask_decay.dev;
    aat::MaskWalk walk;
    HIP_OK(aat::prepare_mask_walk(m == MaskKind::Scan ? aat::kMaskScan : aat::kMaskDense, mask, ps.H, ps.Sq, ps.Sk, t.scan, 0, &walk));
    plain<<<grid, block, T::kSmemBytes, 0>>>(t.q.dev, t.k.dev, t.v.dev, mask, t.o.dev, t.r.dev, ps.H, ps.Sk, ps.Sq, walk.causal, nullptr, walk.extents);
  }
  HIP_OK(hipGetLastError());
  HIP_OK(hipDeviceSynchronize());
}

// Rows of dV, dK (kv positions) and of dQ (query positions) of slice (B-1, H-1) against
//   P = (q k^T) * mask / r,  dV = P^T dO,  dS = (dO v^T) * mask / r,  dK = dS^T q,  dQ = dS k      (r a constant).
static Agreement check_slice(const ProblemShape& ps, Tensors& t, MaskKind m) {
  t.dq.download();
  t.dk.download();
  t.dv.download();
  t.r.download();
  const int bh = ps.B * ps.H - 1, h = ps.H - 1;
  const float gamma = gammas(ps.H)[h];
  const half_t* q = t.q.host.data() + (size_t)bh * ps.Sq * Kd;
  const half_t* k = t.k.host.data() + (size_t)bh * ps.Sk * Kd;
  const half_t* v = t.v.host.data() + (size_t)bh * ps.Sk * D;
  const half_t* g = t.dout.host.data() + (size_t)bh * ps.Sq * D;
  const float* r = t.r.host.data() + (size_t)bh * ps.Sq;
  const half_t* mask = (m == MaskKind::Dense ? t.mask_dense : t.mask_decay).host.data() + (size_t)h * ps.Sq * ps.Sk;
  auto mask_at = [&](int i, int j) {
    return m == MaskKind::Decay ? decay_value(gamma, i + ps.Sk - ps.Sq - j) : (double)(float)mask[(size_t)i * ps.Sk + j];
  };
  auto dot = [](const half_t* a, const half_t* b, int n) {
    double acc = 0;
    for (int c = 0; c < n; ++c) acc += (double)(float)a[c] * (double)(float)b[c];
    return acc;
  };
  Agreement a;
  const int n_rows = 12;
  std::vector<double> dv(D), dk(Kd), dq(Kd);
  for (int n = 0; n < n_rows; ++n) {
    const int j = (int)((long)n * (ps.Sk - 1) / (n_rows - 1));
    std::fill(dv.begin(), dv.end(), 0.0);
    std::fill(dk.begin(), dk.end(), 0.0);
    for (int i = 0; i < ps.Sq; ++i) {
      const double mk = mask_at(i, j);
      if (mk == 0.0) continue;
      const double p = dot(q + (size_t)i * Kd, k + (size_t)j * Kd, Kd) * mk / r[i];
      const double ds = dot(g + (size_t)i * D, v + (size_t)j * D, D) * mk / r[i];
      for (int c = 0; c < D; ++c) dv[c] += p * (double)(float)g[(size_t)i * D + c];
      for (int c = 0; c < Kd; ++c) dk[c] += ds * (double)(float)q[(size_t)i * Kd + c];
    }
    for (int c = 0; c < D; ++c) a.add((double)(float)t.dv.host[((size_t)bh * ps.Sk + j) * D + c], dv[c]);
    for (int c = 0; c < Kd; ++c) a.add((double)(float)t.dk.host[((size_t)bh * ps.Sk + j) * Kd + c], dk[c]);
  }
  for (int n = 0; n < n_rows; ++n) {
    const int i = (int)((long)n * (ps.Sq - 1) / (n_rows - 1));
    std::fill(dq.begin(), dq.end(), 0.0);
    for (int j = 0; j < ps.Sk; ++j) {
      const double mk = mask_at(i, j);
      if (mk == 0.0) continue;
      const double ds = dot(g + (size_t)i * D, v + (size_t)j * D, D) * mk / r[i];
      for (int c = 0; c < Kd; ++c) dq[c] += ds * (double)(float)k[(size_t)j * Kd + c];
    }
    for (int c = 0; c < Kd; ++c) a.add((double)(float)t.dq.host[((size_t)bh * ps.Sq + i) * Kd + c], dq[c]);
  }
  return a;
}

static int g_failures = 0;

// <resident rows, streamed rows per step, threads, buffers of the first-contraction stream, of the second, waves per SIMD>
template <int Br, int Bc, int NT, int NSY, int NSZ, int WPE>
static void test_retnet_bwd(const ProblemShape& ps, Tensors& t) {
  // dV columns per block: the whole row when its accumulators fit the 256 accumulation registers one wave per SIMD
  // has to itself, else 256-column slices over grid.y -- the rule of the per-configuration wrapper.
  constexpr int RTv = Br / (NT / 64) / 32;
  constexpr int DVB = (WPE == 1 && RTv * D <= 512) ? D : 256;
  using TV = aat::RetBwdChain<Kd, D, DVB, Br, Bc, NT, NSY, NSZ, BwdPass::Col>;
  using TK = aat::RetBwdChain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Col>;
  using TQ = aat::RetBwdChain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Row>;
  char name[128];
  std::snprintf(name, sizeof name, "bwd chain Br=%d Bc=%d thr=%d bufs=%d/%d waves/SIMD=%d", Br, Bc, NT, NSY, NSZ, WPE);
  if (ps.Sq % Br || ps.Sk % Br || ps.Sq % Bc || ps.Sk % Bc) {
    std::printf("%-52s skipped: sequence lengths %% %d or %% %d\n", name, Br, Bc);
    return;
  }
  auto dv_plain = &aat::ret_bwd_chain<Kd, D, DVB, Br, Bc, NT, NSY, NSZ, BwdPass::Col, WPE, false>;
  auto dk_plain = &aat::ret_bwd_chain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Col, WPE, false>;
  auto dq_plain = &aat::ret_bwd_chain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Row, WPE, false>;
  auto dv_decay = &aat::ret_bwd_chain<Kd, D, DVB, Br, Bc, NT, NSY, NSZ, BwdPass::Col, WPE, true>;
  auto dk_decay = &aat::ret_bwd_chain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Col, WPE, true>;
  auto dq_decay = &aat::ret_bwd_chain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Row, WPE, true>;
  HIP_OK(hipFuncSetAttribute((const void*)dv_plain, hipFuncAttributeMaxDynamicSharedMemorySize, TV::kSmemBytes));
  HIP_OK(hipFuncSetAttribute((const void*)dv_decay, hipFuncAttributeMaxDynamicSharedMemorySize, TV::kSmemBytes));
  HIP_OK(hipFuncSetAttribute((const void*)dk_plain, hipFuncAttributeMaxDynamicSharedMemorySize, TK::kSmemBytes));
  HIP_OK(hipFuncSetAttribute((const void*)dk_decay, hipFuncAttributeMaxDynamicSharedMemorySize, TK::kSmemBytes));
  HIP_OK(hipFuncSetAttribute((const void*)dq_plain, hipFuncAttributeMaxDynamicSharedMemorySize, TQ::kSmemBytes));
  HIP_OK(hipFuncSetAttribute((const void*)dq_decay, hipFuncAttributeMaxDynamicSharedMemorySize, TQ::kSmemBytes));
  const dim3 block(NT), grid_v(ps.B * ps.H * (ps.Sk / Br), D / DVB), grid_k(ps.B * ps.H * (ps.Sk / Br)), grid_q(ps.B * ps.H * (ps.Sq / Br));
  for (MaskKind m : kAllMasks) {
    if (ps.only && std::strcmp(ps.only, name_of(m))) continue;
    forward_for(ps, t, m);
    const half_t* mask = m == MaskKind::Dense ? t.mask_dense.dev : t.mask_decay.dev;
    auto launch = [&] {
      if (m == MaskKind::Decay) {
        const float* lg = t.log2_gamma.dev;
        dv_decay<<<grid_v, block, TV::kSmemBytes, 0>>>(t.k.dev, t.q.dev, t.dout.dev, nullptr, t.r.dev, t.dv.dev, ps.H, ps.Sk, ps.Sq, 1, lg, nullptr, nullptr);
        dk_decay<<<grid_k, block, TK::kSmemBytes, 0>>>(t.v.dev, t.dout.dev, t.q.dev, nullptr, t.r.dev, t.dk.dev, ps.H, ps.Sk, ps.Sq, 1, lg, nullptr, nullptr);
        dq_decay<<<grid_q, block, TQ::kSmemBytes, 0>>>(t.dout.dev, t.v.dev, t.k.dev, nullptr, t.r.dev, t.dq.dev, ps.H, ps.Sk, ps.Sq, 1, lg, nullptr, nullptr);
        return;
      }
      const int mode = m == MaskKind::Dense ? aat::kMaskDense : m == MaskKind::Causal ? aat::kMaskCausal : aat::kMaskScanned;
      aat::MaskWalk walk;
      HIP_OK(aat::prepare_mask_walk(mode, mask, ps.H, ps.Sq, ps.Sk, t.scan, 0, &walk));
      dv_plain<<<grid_v, block, TV::kSmemBytes, 0>>>(t.k.dev, t.q.dev, t.dout.dev, mask, t.r.dev, t.dv.dev, ps.H, ps.Sk, ps.Sq, walk.causal, nullptr, walk.extents, nullptr);
      dk_plain<<<grid_k, block, TK::kSmemBytes, 0>>>(t.v.dev, t.dout.dev, t.q.dev, mask, t.r.dev, t.dk.dev, ps.H, ps.Sk, ps.Sq, walk.causal, nullptr, walk.extents, nullptr);
      dq_plain<<<grid_q, block, TQ::kSmemBytes, 0>>>(t.dout.dev, t.v.dev, t.k.dev, mask, t.r.dev, t.dq.dev, ps.H, ps.Sk, ps.Sq, walk.causal, nullptr, walk.extents, nullptr);
    };
    for (auto* x : {&t.dq, &t.dk, &t.dv}) HIP_OK(hipMemset(x->dev, 0xff, x->host.size() * sizeof(half_t)));
    launch();
    HIP_OK(hipGetLastError());
    HIP_OK(hipDeviceSynchronize());
    const Agreement agree = check_slice(ps, t, m);
    g_failures += !agree.ok();
    const aat_bench::Timing tm = aat_bench::do_bench(launch, ps.flush);
    const double fl = 2.0 * ps.B * ps.H * (double)ps.Sq * ps.Sk * (3 * Kd + 2 * D) * share_of_dense(m);
    std::printf("%-52s mask %-6s mean %.4f ms  median %.4f  p20 %.4f  p80 %.4f  (%d launches)  %.1f TFLOP/s = %.1f%% of 2.5 PFLOP/s"
                "  check: max |err| %.2e of %.2f -> %s\n", name, name_of(m), tm.mean_ms, tm.median_ms, tm.p20_ms, tm.p80_ms, tm.launches,
                fl / tm.median_ms * 1e-9, fl / tm.median_ms * 1e-9 / 25.0, agree.max_err, agree.max_ref, agree.ok() ? "ok" : "MISMATCH");
  }
}

// The same with dS stored by the row pass and read back by a dK kernel of its own
// <resident rows, streamed rows, threads, Y/Z buffers of the chained passes; kv rows, query rows, threads, stages, waves per SIMD of the dK kernel>
template <int Br, int Bc, int NT, int NSY, int NSZ, int KBX, int KBY, int KNT, int KNS, int KWPE>
static void test_retnet_bwd_stored_ds(const ProblemShape& ps, Tensors& t) {
  constexpr int WPE = 1;
  constexpr int RTv = Br / (NT / 64) / 32;
  constexpr int DVB = (WPE == 1 && RTv * D <= 512) ? D : 256;
  using TV = aat::RetBwdChain<Kd, D, DVB, Br, Bc, NT, NSY, NSZ, BwdPass::Col>;
  using TQ = aat::RetBwdChain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Row>;
  using TK = aat::RetBwdDk<Kd, KBX, KBY, KNT, KNS>;
  static_assert(Br % KBY == 0, "a query tile of the dK kernel lies inside one block of the row pass");
  char name[160];
  std::snprintf(name, sizeof name, "bwd chain Br=%d Bc=%d thr=%d bufs=%d/%d waves/SIMD=%d dK from dS %dx%d", Br, Bc, NT, NSY, NSZ, WPE, KBX, KBY);
  if (ps.Sq % Br || ps.Sk % Br || ps.Sq % Bc || ps.Sk % Bc || ps.Sk % KBX || ps.Sq % KBY) {
    std::printf("%-70s skipped: sequence lengths\n", name);
    return;
  }
  auto dv_plain = &aat::ret_bwd_chain<Kd, D, DVB, Br, Bc, NT, NSY, NSZ, BwdPass::Col, WPE, false>;
  auto dq_plain = &aat::ret_bwd_chain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Row, WPE, false, true>;
  auto dv_decay = &aat::ret_bwd_chain<Kd, D, DVB, Br, Bc, NT, NSY, NSZ, BwdPass::Col, WPE, true>;
  auto dq_decay = &aat::ret_bwd_chain<D, Kd, Kd, Br, Bc, NT, NSY, NSZ, BwdPass::Row, WPE, true, true>;
  auto dk_ds = &aat::ret_bwd_dk_from_ds<Kd, KBX, KBY, KNT, KNS, KWPE>;
  HIP_OK(hipFuncSetAttribute((const void*)dv_plain, hipFuncAttributeMaxDynamicSharedMemorySize, TV::kSmemBytes));
  HIP_OK(hipFuncSetAttribute((const void*)dv_decay, hipFuncAttributeMaxDynamicSharedMemorySize, TV::kSmemBytes));
  HIP_OK(hipFuncSetAttribute((const void*)dq_plain, hipFuncAttributeMaxDynamicSharedMemorySize, TQ::kSmemBytesDsOut));
  HIP_OK(hipFuncSetAttribute((const void*)dq_decay, hipFuncAttributeMaxDynamicSharedMemorySize, TQ::kSmemBytesDsOut));
  HIP_OK(hipFuncSetAttribute((const void*)dk_ds, hipFuncAttributeMaxDynamicSharedMemorySize, TK::kSmemBytes));
  const dim3 block(NT), grid_v(ps.B * ps.H * (ps.Sk / Br), D / DVB), grid_q(ps.B * ps.H * (ps.Sq / Br));
  const dim3 kblock(KNT), grid_k(ps.B * ps.H * (ps.Sk / KBX));
  for (MaskKind m : kAllMasks) {
    if (ps.only && std::strcmp(ps.only, name_of(m))) continue;
    forward_for(ps, t, m);
    const half_t* mask = m == MaskKind::Dense ? t.mask_dense.dev : t.mask_decay.dev;
    auto launch = [&] {
      if (m == MaskKind::Decay) {
        const float* lg = t.log2_gamma.dev;
        dv_decay<<<grid_v, block, TV::kSmemBytes, 0>>>(t.k.dev, t.q.dev, t.dout.dev, nullptr, t.r.dev, t.dv.dev, ps.H, ps.Sk, ps.Sq, 1, lg, nullptr, nullptr);
        dq_decay<<<grid_q, block, TQ::kSmemBytesDsOut, 0>>>(t.dout.dev, t.v.dev, t.k.dev, nullptr, t.r.dev, t.dq.dev, ps.H, ps.Sk, ps.Sq, 1, lg, nullptr, t.ds);
        dk_ds<<<grid_k, kblock, TK::kSmemBytes, 0>>>(t.q.dev, t.ds, t.dk.dev, ps.H, ps.Sk, ps.Sq, 1, nullptr, Br, Bc);
        return;
      }
      const int mode = m == MaskKind::Dense ? aat::kMaskDense : m == MaskKind::Causal ? aat::kMaskCausal : aat::kMaskScanned;
      aat::MaskWalk walk;
      HIP_OK(aat::prepare_mask_walk(mode, mask, ps.H, ps.Sq, ps.Sk, t.scan, 0, &walk));
      dv_plain<<<grid_v, block, TV::kSmemBytes, 0>>>(t.k.dev, t.q.dev, t.dout.dev, mask, t.r.dev, t.dv.dev, ps.H, ps.Sk, ps.Sq, walk.causal, nullptr, walk.extents, nullptr);
      dq_plain<<<grid_q, block, TQ::kSmemBytesDsOut, 0>>>(t.dout.dev, t.v.dev, t.k.dev, mask, t.r.dev, t.dq.dev, ps.H, ps.Sk, ps.Sq, walk.causal, nullptr, walk.extents, t.ds);
      dk_ds<<<grid_k, kblock, TK::kSmemBytes, 0>>>(t.q.dev, t.ds, t.dk.dev, ps.H, ps.Sk, ps.Sq, walk.causal, walk.extents, Br, Bc);
    };
    for (auto* x : {&t.dq, &t.dk, &t.dv}) HIP_OK(hipMemset(x->dev, 0xff, x->host.size() * sizeof(half_t)));
    HIP_OK(hipMemset(t.ds, 0x7f, (size_t)ps.B * ps.H * ps.Sq * ps.Sk * sizeof(half_t)));     // NaN patterns where nothing is written
    launch();
    HIP_OK(hipGetLastError());
    HIP_OK(hipDeviceSynchronize());
    const Agreement agree = check_slice(ps, t, m);
    g_failures += !agree.ok();
    const aat_bench::Timing tm = aat_bench::do_bench(launch, ps.flush);
    const double fl = 2.0 * ps.B * ps.H * (double)ps.Sq * ps.Sk * (3 * Kd + 2 * D) * share_of_dense(m);
    std::printf("%-70s mask %-6s mean %.4f ms  median %.4f  p20 %.4f  p80 %.4f  (%d launches)  %.1f TFLOP/s = %.1f%% of 2.5 PFLOP/s"
                "  check: max |err| %.2e of %.2f -> %s\n", name, name_of(m), tm.mean_ms, tm.median_ms, tm.p20_ms, tm.p80_ms, tm.launches,
                fl / tm.median_ms * 1e-9, fl / tm.median_ms * 1e-9 / 25.0, agree.max_err, agree.max_ref, agree.ok() ? "ok" : "MISMATCH");
  }
}

int main(int argc, char** argv) {
  ProblemShape ps;
  if (!parse_args(argc, argv, &ps)) {
    std::printf("usage: %s [B H Sq Sk] [--mask dense|causal|scan|decay] [--no-flush]\n", argv[0]);
    return 2;
  }
  if (ps.Sq % 128 || ps.Sk % 64) {
    std::printf("the forward that supplies r needs Sq %% 128 == 0 and Sk %% 64 == 0\n");
    return 2;
  }
  hipDeviceProp_t prop;
  HIP_OK(hipGetDeviceProperties(&prop, 0));
  std::printf("%s  %d CUs  LDS/block %zu KB   RetNet backward B=%d H=%d Sq=%d Sk=%d d_qk=%d d_v=%d fp16 %s\n", prop.gcnArchName,
              prop.multiProcessorCount, prop.sharedMemPerBlockOptin / 1024, ps.B, ps.H, ps.Sq, ps.Sk, Kd, D,
              ps.flush ? "(cache flushed before every launch)" : "(hot cache)");
  Tensors t;
  const size_t nq = (size_t)ps.B * ps.H * ps.Sq * Kd, nk = (size_t)ps.B * ps.H * ps.Sk * Kd;
  const size_t nv = (size_t)ps.B * ps.H * ps.Sk * D, no = (size_t)ps.B * ps.H * ps.Sq * D;
  t.q = randn(nq, 1);
  t.k = randn(nk, 2);
  t.v = randn(nv, 3);
  t.mask_dense = randn((size_t)ps.H * ps.Sq * ps.Sk, 4);
  t.dout = randn(no, 5);
  t.mask_decay = decay_mask(ps.H, ps.Sq, ps.Sk);
  t.log2_gamma = log2_gammas(ps.H);
  t.o = empty<half_t>(no);
  t.r = empty<float>((size_t)ps.B * ps.H * ps.Sq);
  t.dq = empty<half_t>(nq);
  t.dk = empty<half_t>(nk);
  t.dv = empty<half_t>(nv);
  HIP_OK(hipMalloc(&t.scan, aat::mask_extent_bytes(ps.H, ps.Sq, ps.Sk)));
  HIP_OK(hipMalloc(&t.ds, (size_t)ps.B * ps.H * ps.Sq * ps.Sk * sizeof(half_t)));

  test_retnet_bwd_stored_ds<128, 64, 256, 1, 1, 128, 64, 256, 2, 2>(ps, t);
  test_retnet_bwd_stored_ds<128, 32, 256, 1, 1, 256, 64, 512, 2, 2>(ps, t);
  test_retnet_bwd_stored_ds<128, 64, 256, 1, 1, 256, 64, 512, 2, 2>(ps, t);
  test_retnet_bwd<128, 32, 256, 3, 2, 1>(ps, t);
  test_retnet_bwd<128, 64, 256, 1, 1, 1>(ps, t);
  test_retnet_bwd<128, 32, 256, 2, 2, 1>(ps, t);

  for (auto* x : {&t.q, &t.k, &t.v, &t.dout, &t.mask_dense, &t.mask_decay, &t.o, &t.dq, &t.dk, &t.dv}) x->release();
  t.r.release();
  t.log2_gamma.release();
  HIP_OK(hipFree(t.scan));
  HIP_OK(hipFree(t.ds));
  if (g_failures) std::printf("%d result(s) disagree with the host formulas\n", g_failures);
  return g_failures ? 1 : 0;
}
