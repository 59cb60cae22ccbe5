// What the two stand-alone RetNet benchmarks share: synthetic inputs, the four ways of handing the mask to a
// kernel, and the plain formulas on the host that one (batch, head) slice of every result is checked against
// (reference python/utils/ref_op.py:8-13 for the forward; the gradients are those of that expression with r held
// constant, as reference csrc/kernels/retnet/bwd/bwd_colblock.h:509,551 computes them).
#pragma once
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../kernels/utils/mask_extents.h"
#include "do_bench.h"

#define HIP_OK(x)                                                                     \
  do {                                                                                \
    hipError_t e_ = (x);                                                              \
    if (e_ != hipSuccess) {                                                           \
      std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(1);                                                                   \
    }                                                                                 \
  } while (0)

namespace retnet_bench {

using half_t = aat::half_t;

struct ProblemShape {
  int B = 4, H = 8, Sq = 2048, Sk = 2048;      // reference benchmarks/retnet/retnet.cu:218: ProblemShape PS(4,8,2048,2048)
  bool flush = true;
  const char* only = nullptr;                  // --mask <name>: time this mask mode only
};

// How the mask reaches the kernel.
//   dense   N(0,1) mask tensor, every tile walked (what the reference's benchmark times)
//   causal  RetNet's decay mask as a tensor, zeros above the diagonal promised by the caller
//   scan    the same tensor, its non-zero ranges found by a scan on the GPU that is part of the timed launch
//   decay   no tensor: gamma_h per head, the mask built in registers
enum class MaskKind { Dense, Causal, Scan, Decay };
inline const char* name_of(MaskKind m) {
  switch (m) {
    case MaskKind::Dense: return "dense";
    case MaskKind::Causal: return "causal";
    case MaskKind::Scan: return "scan";
    default: return "decay";
  }
}
constexpr MaskKind kAllMasks[] = {MaskKind::Dense, MaskKind::Causal, MaskKind::Scan, MaskKind::Decay};

inline bool parse_args(int argc, char** argv, ProblemShape* ps) {
  int pos = 0;
  for (int i = 1; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--no-flush")) ps->flush = false;
    else if (!std::strcmp(argv[i], "--mask") && i + 1 < argc) ps->only = argv[++i];
    else if (argv[i][0] == '-') return false;
    else {
      const int v = std::atoi(argv[i]);
      if (pos == 0) ps->B = v; else if (pos == 1) ps->H = v; else if (pos == 2) ps->Sq = v; else if (pos == 3) ps->Sk = v;
      ++pos;
    }
  }
  if (ps->only) {
    bool known = false;
    for (MaskKind m : kAllMasks) known |= !std::strcmp(ps->only, name_of(m));
    if (!known) return false;
  }
  return ps->B > 0 && ps->H > 0 && ps->Sq > 0 && ps->Sk > 0;
}

template <class T> struct HostDevice {
  std::vector<T> host;
  T* dev = nullptr;
  void upload() {
    HIP_OK(hipMalloc(&dev, host.size() * sizeof(T)));
    HIP_OK(hipMemcpy(dev, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
  }
  void download() { HIP_OK(hipMemcpy(host.data(), dev, host.size() * sizeof(T), hipMemcpyDeviceToHost)); }
  void release() {
    if (dev) HIP_OK(hipFree(dev));
    dev = nullptr;
  }
};

inline HostDevice<half_t> randn(size_t n, unsigned seed) {
  HostDevice<half_t> t;
  t.host.resize(n);
  std::mt19937 gen(seed);
  std::normal_distribution<float> dist(0.f, 1.f);
  for (auto& x : t.host) x = (half_t)dist(gen);
  t.upload();
  return t;
}
template <class T> inline HostDevice<T> empty(size_t n) {
  HostDevice<T> t;
  t.host.resize(n);
  HIP_OK(hipMalloc(&t.dev, n * sizeof(T)));
  HIP_OK(hipMemset(t.dev, 0xff, n * sizeof(T)));
  return t;
}

// RetNet's rates: gamma_h = 1 - 2^(-5-h).
inline std::vector<float> gammas(int H) {
  std::vector<float> g(H);
  for (int h = 0; h < H; ++h) g[h] = 1.f - std::exp2(-5.f - (float)h);
  return g;
}
// mask[h][i][j] = gamma_h^(i + Sk - Sq - j) on and below that diagonal, 0 above it, rounded to fp16.
inline HostDevice<half_t> decay_mask(int H, int Sq, int Sk) {
  HostDevice<half_t> t;
  t.host.resize((size_t)H * Sq * Sk);
  const std::vector<float> g = gammas(H);
  for (int h = 0; h < H; ++h) {
    std::vector<half_t> power(Sq + Sk);
    for (int e = 0; e < Sq + Sk; ++e) power[e] = (half_t)std::pow((double)g[h], (double)e);
    for (int i = 0; i < Sq; ++i)
      for (int j = 0; j < Sk; ++j) {
        const int e = i + Sk - Sq - j;
        t.host[((size_t)h * Sq + i) * Sk + j] = e >= 0 ? power[e] : (half_t)0.f;
      }
  }
  t.upload();
  return t;
}
inline HostDevice<float> log2_gammas(int H) {
  HostDevice<float> t;
  for (float g : gammas(H)) t.host.push_back(std::log2(g));
  t.upload();
  return t;
}
// The value of the register-built mask at exponent e: fp32 in the kernels, never rounded to fp16.
inline double decay_value(float gamma, int e) { return e >= 0 ? std::pow((double)gamma, (double)e) : 0.0; }

// What every kernel of a benchmark is launched with for one mask kind.
struct MaskArgs {
  const half_t* mask = nullptr;       // tensor, or nullptr for Decay
  const float* log2_gamma = nullptr;  // Decay only
  int walk_mode = aat::kMaskDense;    // what prepare_mask_walk is called with before the kernels
  void* workspace = nullptr;          // Scan: room for the non-zero ranges
};

inline double share_of_dense(MaskKind m) { return m == MaskKind::Dense ? 1.0 : 0.5; }

// One entry of a result against its fp32-exact value: 2e-3 absolute for small values and the fp16 spacing for
// large ones, doubled -- this is a check that the benchmark launches what it says, not the parity gate.
struct Agreement {
  double max_err = 0, max_ref = 0;
  long bad = 0, n = 0;
  void add(double got, double ref) {
    const double err = std::fabs(got - ref);
    max_err = std::max(max_err, err);
    max_ref = std::max(max_ref, std::fabs(ref));
    bad += !(err <= 4e-3 + std::fabs(ref) * (1.0 / 512));
    ++n;
  }
  bool ok() const { return n > 0 && bad == 0; }
};

}  // namespace retnet_bench
