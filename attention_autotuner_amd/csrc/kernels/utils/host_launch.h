// Host-side helpers shared by the generated per-configuration wrappers: shape checks, dynamic-LDS
// opt-in and the self-calibrating timing loop behind `profile`.
//
// The timing protocol is the reference's (reference: csrc/kernels/attention/regfuse/profile_code.py:36-63):
// one timed launch to estimate t, then ceil(100 ms / t) back-to-back launches between two events, mean
// time per launch returned, -1 on any runtime error.
#pragma once
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdio>

namespace aat {

inline bool shape_ok(int B, int H, int Seq_q, int Seq_k, int Br, int Bc) {
  return B > 0 && H > 0 && Seq_q > 0 && Seq_k > 0 && Seq_q % Br == 0 && Seq_k % Bc == 0;
}

// Kernels here use more than the 64 KB of LDS a launch gets by default; opt in once per kernel.
template <class K> inline hipError_t allow_lds(K kernel, int bytes) {
  if (bytes <= 64 * 1024) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

// `launch()` enqueues one complete invocation on `stream` and returns a hipError_t.
template <class F> inline float timed_mean_ms(hipStream_t stream, F launch) {
  hipEvent_t start, stop;
  if (hipEventCreate(&start) != hipSuccess) return -1.f;
  if (hipEventCreate(&stop) != hipSuccess) { (void)hipEventDestroy(start); return -1.f; }
  float ms = -1.f;
  bool ok = false;
  do {
    if (hipEventRecord(start, stream) != hipSuccess) break;
    if (launch() != hipSuccess) break;
    if (hipEventRecord(stop, stream) != hipSuccess) break;
    if (hipEventSynchronize(stop) != hipSuccess) break;
    if (hipGetLastError() != hipSuccess) break;
    if (hipEventElapsedTime(&ms, start, stop) != hipSuccess) break;
    int repeats = (int)std::ceil(100.0 / (ms > 1e-4f ? ms : 1e-4f));
    if (repeats < 1) repeats = 1;
    if (repeats > 20000) repeats = 20000;
    if (hipEventRecord(start, stream) != hipSuccess) break;
    bool launched = true;
    for (int i = 0; i < repeats; ++i)
      if (launch() != hipSuccess) { launched = false; break; }
    if (!launched) break;
    if (hipEventRecord(stop, stream) != hipSuccess) break;
    if (hipEventSynchronize(stop) != hipSuccess) break;
    if (hipGetLastError() != hipSuccess) break;
    if (hipEventElapsedTime(&ms, start, stop) != hipSuccess) break;
    ms /= repeats;
    ok = true;
  } while (false);
  (void)hipEventDestroy(start);
  (void)hipEventDestroy(stop);
  if (!ok) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) std::printf("HIP error: %s\n", hipGetErrorString(e));
    return -1.f;
  }
  return ms;
}

}  // namespace aat
