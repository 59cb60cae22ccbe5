// Stand-alone benchmark of the RetNet recurrent form: calls the library's `retnet_recurrent_fwd` exactly as
// the reference's benchmark calls its own (reference benchmarks/retnet/retnet.cu:173-215, shape :236), and
// checks one (batch, head) slice against the plain recurrence on the host.
//
//   hipcc --offload-arch=gfx950 -O3 -I attention_autotuner_amd/csrc \
//         attention_autotuner_amd/csrc/benchmarks/retnet_recurrent.hip -ldl -o retnet_recurrent_bench
//   ./retnet_recurrent_bench <path to ret_recurrent_*.so> [B H L dim_qk dim_v] [--no-flush]
//
// The library is opened with dlopen so that the same binary serves every build of it; linking it in
// (-l:ret_recurrent_r1-<digest>.so) works the same way, the symbol and its arguments are the reference's.
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "do_bench.h"

#define HIP_OK(x)                                                                     \
  do {                                                                                \
    hipError_t e_ = (x);                                                              \
    if (e_ != hipSuccess) {                                                           \
      std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(1);                                                                   \
    }                                                                                 \
  } while (0)

using recurrent_fn = void (*)(void*, void*, void*, void*, void*, int, int, int, int, int, int);

static float* device_uniform(size_t n, unsigned seed, float lo, float hi, std::vector<float>* keep = nullptr) {
  std::vector<float> h(n);
  std::mt19937 gen(seed);
  std::uniform_real_distribution<float> u(lo, hi);
  for (auto& x : h) x = u(gen);
  float* d = nullptr;
  HIP_OK(hipMalloc(&d, n * sizeof(float)));
  HIP_OK(hipMemcpy(d, h.data(), n * sizeof(float), hipMemcpyHostToDevice));
  if (keep) keep->swap(h);
  return d;
}

int main(int argc, char** argv) {
  if (argc < 2) {
    std::printf("usage: %s <ret_recurrent library> [B H L dim_qk dim_v] [--no-flush]\n", argv[0]);
    return 2;
  }
  int B = 8, H = 32, L = 2048, dim_qk = 128, dim_v = 128;      // recurrentShape PS2(8,32,2048,2048,128,128)
  bool flush = true;
  std::vector<int> nums;
  for (int i = 2; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--no-flush")) flush = false;
    else nums.push_back(std::atoi(argv[i]));
  }
  if (nums.size() == 5) { B = nums[0]; H = nums[1]; L = nums[2]; dim_qk = nums[3]; dim_v = nums[4]; }
  void* lib = dlopen(argv[1], RTLD_NOW);
  if (!lib) { std::printf("dlopen failed: %s\n", dlerror()); return 1; }
  auto fn = reinterpret_cast<recurrent_fn>(dlsym(lib, "retnet_recurrent_fwd"));
  if (!fn) { std::printf("retnet_recurrent_fwd not found in %s\n", argv[1]); return 1; }

  const size_t nq = (size_t)B * H * L * dim_qk, nv = (size_t)B * H * L * dim_v;
  std::vector<float> hq, hk, hv, hd;
  float* q = device_uniform(nq, 1, -1.f, 1.f, &hq);
  float* k = device_uniform(nq, 2, -1.f, 1.f, &hk);
  float* v = device_uniform(nv, 3, -1.f, 1.f, &hv);
  float* decay = device_uniform((size_t)H * L, 4, 0.9f, 1.f, &hd);
  float* out = nullptr;
  HIP_OK(hipMalloc(&out, nv * sizeof(float)));
  HIP_OK(hipMemset(out, 0xff, nv * sizeof(float)));

  fn(q, k, v, decay, out, B, H, dim_qk, dim_v, L, dim_qk);
  HIP_OK(hipDeviceSynchronize());

  // host check: slice (B-1, H-1), every value dim, plain recurrence in double
  {
    const int bh = B * H - 1, h = H - 1;
    std::vector<float> ho((size_t)dim_v * L);
    HIP_OK(hipMemcpy(ho.data(), out + (size_t)bh * dim_v * L, ho.size() * sizeof(float), hipMemcpyDeviceToHost));
    std::vector<double> S((size_t)dim_qk * dim_v, 0.0);
    double max_err = 0, max_ref = 0;
    for (int n = 0; n < L; ++n) {
      const double a = hd[(size_t)h * L + n];
      for (int kd = 0; kd < dim_qk; ++kd) {
        const double kk = hk[((size_t)bh * dim_qk + kd) * L + n];
        for (int vd = 0; vd < dim_v; ++vd)
          S[(size_t)kd * dim_v + vd] = a * S[(size_t)kd * dim_v + vd] + kk * hv[((size_t)bh * dim_v + vd) * L + n];
      }
      for (int vd = 0; vd < dim_v; ++vd) {
        double acc = 0;
        for (int kd = 0; kd < dim_qk; ++kd) acc += (double)hq[((size_t)bh * dim_qk + kd) * L + n] * S[(size_t)kd * dim_v + vd];
        max_err = std::max(max_err, std::fabs(acc - (double)ho[(size_t)vd * L + n]));
        max_ref = std::max(max_ref, std::fabs(acc));
      }
    }
    std::printf("check (batch %d, head %d): max |err| %.3e, max |ref| %.3e -> %s\n", B - 1, H - 1, max_err, max_ref,
                max_err <= 2e-5 * max_ref ? "ok" : "MISMATCH");
    if (!(max_err <= 2e-5 * max_ref)) return 1;
  }

  const aat_bench::Timing t = aat_bench::do_bench([&]() { fn(q, k, v, decay, out, B, H, dim_qk, dim_v, L, dim_qk); }, flush);
  const double flops = 5.0 * B * H * (double)L * dim_qk * dim_v;     // two multiply-adds and one multiply per (position, kd, vd)
  const double bytes = 4.0 * (2.0 * nq + 2.0 * nv);
  std::printf("retnet_recurrent_fwd B=%d H=%d L=%d dim_qk=%d dim_v=%d: mean %.4f ms, median %.4f (p20 %.4f, p80 %.4f, %d launches)"
              " -> %.1f TFLOP/s, %.2f TB/s\n", B, H, L, dim_qk, dim_v, t.mean_ms, t.median_ms, t.p20_ms, t.p80_ms, t.launches,
              flops / t.median_ms * 1e-9, bytes / t.median_ms * 1e-9);
  return 0;
}
