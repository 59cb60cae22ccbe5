// Timing protocol of the stand-alone benchmark (reference: benchmarks/do_bench.cuh:8-63): estimate with five
// launches, warm up for ~50 ms, measure for ~100 ms with one event pair per launch and a 256 MB
// write before every timed launch so no input survives in L2 / MALL between launches.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <functional>
#include <vector>

namespace aat_bench {

struct Timing {
  float mean_ms, median_ms, p20_ms, p80_ms;
  int launches;
};

__global__ void flush_fill(int* p, size_t n, int value) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = value;
}

inline Timing do_bench(const std::function<void()>& launch, bool flush_cache = true, int ms_warmup = 50, int ms_measure = 100) {
  const size_t n_flush = (size_t)(256e6 / 4);
  int* cache = nullptr;
  if (flush_cache && hipMalloc(&cache, n_flush * sizeof(int)) != hipSuccess) cache = nullptr;
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  launch();
  (void)hipEventRecord(e0, 0);
  for (int i = 0; i < 5; ++i) launch();
  (void)hipEventRecord(e1, 0);
  (void)hipEventSynchronize(e1);
  float est = 0.f;
  (void)hipEventElapsedTime(&est, e0, e1);
  est = std::max(est / 5.f, 1e-4f);
  const int warm = std::max(1, (int)std::ceil(ms_warmup / est));
  const int measure = std::min(20000, std::max(1, (int)std::ceil(ms_measure / est)));
  for (int i = 0; i < warm; ++i) launch();
  std::vector<hipEvent_t> s(measure), t(measure);
  for (int i = 0; i < measure; ++i) {
    (void)hipEventCreate(&s[i]);
    (void)hipEventCreate(&t[i]);
  }
  for (int i = 0; i < measure; ++i) {
    if (cache) flush_fill<<<2048, 256>>>(cache, n_flush, i);
    (void)hipEventRecord(s[i], 0);
    launch();
    (void)hipEventRecord(t[i], 0);
  }
  if (hipDeviceSynchronize() != hipSuccess) std::printf("HIP error: %s\n", hipGetErrorString(hipGetLastError()));
  std::vector<float> ms(measure);
  for (int i = 0; i < measure; ++i) {
    (void)hipEventElapsedTime(&ms[i], s[i], t[i]);
    (void)hipEventDestroy(s[i]);
    (void)hipEventDestroy(t[i]);
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (cache) (void)hipFree(cache);
  Timing out;
  out.launches = measure;
  out.mean_ms = 0.f;
  for (float x : ms) out.mean_ms += x;
  out.mean_ms /= measure;
  std::sort(ms.begin(), ms.end());
  out.median_ms = ms[measure / 2];
  out.p20_ms = ms[(size_t)(0.2 * (measure - 1))];
  out.p80_ms = ms[(size_t)(0.8 * (measure - 1))];
  return out;
}

}  // namespace aat_bench
