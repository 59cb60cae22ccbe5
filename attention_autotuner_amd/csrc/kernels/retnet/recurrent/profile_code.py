"""Source text of the wrapper library for the RetNet recurrent form
(same role as the ``extern "C" retnet_recurrent_fwd`` at the end of reference
csrc/kernels/retnet/recurrent/recurrent.h:427-463, which the reference compiles straight into its
benchmark, benchmarks/retnet/retnet.cu:175-215).

One library holds every supported (key dims, value slice) instantiation and picks one per call, so the
only field of the configuration record is a revision tag.
"""

global_vars = r"""
#define AAT_OP_RET_RECURRENT 1
#include "aat_kernel_abi.h"
#include "kernels/retnet/recurrent/recurrent.h"
#include "kernels/utils/host_launch.h"
#include <mutex>

namespace {{
constexpr int kRevision = {revision};

constexpr int kMaxKdim = 256;                     // the reference's MAX_KDIM (reference recurrent.h:18)

size_t factor_bytes(int heads, int l) {{ return (size_t)heads * (size_t)(l / 32) * aat::kRecFactorBytes; }}
// More than 128 key dims are contracted in passes of 128 (or 64) whose outputs add; every pass but the
// first writes into a second output-sized buffer behind the decay factors.
size_t total_workspace_bytes(int batch, int heads, int vdim, int l, int block_kdim) {{
  const size_t f = (factor_bytes(heads, l) + 255) / 256 * 256;
  return block_kdim > 128 ? f + (size_t)batch * heads * vdim * l * sizeof(float) : f;
}}

bool rec_shape_ok(int batch, int heads, int kdim, int vdim, int l, int block_kdim) {{
  return batch > 0 && heads > 0 && l > 0 && l % 32 == 0 && l / 32 <= 4096 && block_kdim >= 64 && block_kdim % 64 == 0 &&
         block_kdim <= kMaxKdim && block_kdim <= kdim && vdim > 0 && vdim % 64 == 0;
}}

__global__ void rec_add_kernel(float4* __restrict__ out, const float4* __restrict__ part, size_t n4) {{
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {{
    float4 a = out[i];
    const float4 b = part[i];
    a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    out[i] = a;
  }}
}}

template <int KD, int DVS>
hipError_t launch_one(const float* q, const float* k, const float* v, const char* factors, float* out, int batch,
                      int heads, int kdim, int vdim, int l, hipStream_t stream) {{
  using T = aat::RetRecurrent<KD, DVS>;
  const auto kernel = &aat::retnet_recurrent_kernel<KD, DVS>;
  static const hipError_t ok = aat::allow_lds(kernel, T::kSmemBytes);
  if (ok != hipSuccess) return ok;
  kernel<<<dim3(vdim / DVS, batch * heads), dim3(T::kThreads), T::kSmemBytes, stream>>>(q, k, v, factors, out, heads,
                                                                                    kdim, vdim, l);
  return hipGetLastError();
}}

// Two launches: the decay factors of every (head, chunk), then the scan.  A value slice of 128 dims per
// block halves the traffic of q and k; 64 is taken when vdim asks for it or when 128 would leave most of
// the compute units without a block.
hipError_t launch(const float* q, const float* k, const float* v, const float* decay, float* out, int batch, int heads,
                  int kdim, int vdim, int l, int block_kdim, char* workspace, hipStream_t stream) {{
  char* factors = workspace;
  float* part = reinterpret_cast<float*>(workspace + (factor_bytes(heads, l) + 255) / 256 * 256);
  aat::retnet_recurrent_factors<<<dim3(heads), dim3(aat::kRecFactorThreads), (size_t)(l / 32) * 16, stream>>>(decay, factors, l);
  hipError_t e = hipGetLastError();
  const bool wide = vdim % 128 == 0 && (long)batch * heads * (vdim / 128) >= 192;
  for (int kd0 = 0; kd0 < block_kdim && e == hipSuccess; ) {{
    const int kd = block_kdim - kd0 >= 128 ? 128 : 64;                 // key dims of this pass
    const float* qp = q + (size_t)kd0 * l;                             // rows kd0.. of every (batch, head) slice
    const float* kp = k + (size_t)kd0 * l;
    float* dst = kd0 == 0 ? out : part;
    if (kd == 128)
      e = wide ? launch_one<128, 128>(qp, kp, v, factors, dst, batch, heads, kdim, vdim, l, stream)
               : launch_one<128, 64>(qp, kp, v, factors, dst, batch, heads, kdim, vdim, l, stream);
    else
      e = wide ? launch_one<64, 128>(qp, kp, v, factors, dst, batch, heads, kdim, vdim, l, stream)
               : launch_one<64, 64>(qp, kp, v, factors, dst, batch, heads, kdim, vdim, l, stream);
    if (e == hipSuccess && kd0 > 0) {{
      const size_t n4 = (size_t)batch * heads * vdim * l / 4;
      rec_add_kernel<<<dim3(2048), dim3(256), 0, stream>>>(reinterpret_cast<float4*>(out), reinterpret_cast<const float4*>(part), n4);
      e = hipGetLastError();
    }}
    kd0 += kd;
  }}
  return e;
}}

// Workspace of the reference-signature entry point, which has no argument to bring one in: one buffer
// per device, grown on demand, kept until the process ends.
std::mutex g_ws_mutex;
struct DeviceWorkspace {{ char* ptr = nullptr; size_t bytes = 0; }};
DeviceWorkspace g_ws[64];

char* cached_workspace(size_t bytes) {{
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  DeviceWorkspace& w = g_ws[dev];
  if (w.bytes < bytes) {{
    if (w.ptr != nullptr) {{
      if (hipDeviceSynchronize() != hipSuccess) return nullptr;     // earlier launches may still read it
      (void)hipFree(w.ptr);
      w.ptr = nullptr;
      w.bytes = 0;
    }}
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) return nullptr;
    w.ptr = static_cast<char*>(p);
    w.bytes = bytes;
  }}
  return w.ptr;
}}

// The entry point that allocates nothing keeps its decay factors in device memory that is part of this
// library's code object: one copy of `scratch` per device that loads the library, held until the process ends.
constexpr size_t kNoAllocScratchBytes = (size_t)AAT_RECURRENT_NOALLOC_MAX_RECORDS * aat::kRecFactorBytes;
}}  // namespace

static __device__ __align__(256) char scratch[kNoAllocScratchBytes];

namespace {{
// In host code `scratch` is only a handle for hipGetSymbolAddress; the device address differs per device
// and is looked up once for each, with that device current.
std::mutex g_scratch_mutex;
char* g_scratch_ptr[64];

hipError_t scratch_of_current_device(char** ptr) {{
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {{
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (p == nullptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = static_cast<char*>(p);
  }}
  *ptr = g_scratch_ptr[dev];
  return hipSuccess;
}}
}}  // namespace
"""

kernel_code = global_vars + r"""
extern "C" int abi_version(void) {{ return AAT_ABI_VERSION; }}
extern "C" const char* config_string(void) {{ return "{config_name}"; }}
extern "C" size_t workspace_size(int B, int H, int Seq_q, int Seq_k) {{
  (void)B; (void)Seq_k;                           // up to 128 key dims; retnet_recurrent_workspace_size covers every case
  return H > 0 && Seq_q > 0 ? (factor_bytes(H, Seq_q) + 255) / 256 * 256 : 0;
}}

extern "C" size_t retnet_recurrent_workspace_size(int batch, int heads, int kdim, int vdim, int l, int block_kdim) {{
  return rec_shape_ok(batch, heads, kdim, vdim, l, block_kdim) ? total_workspace_bytes(batch, heads, vdim, l, block_kdim) : 0;
}}

extern "C" int retnet_recurrent_fwd_ex(const float* q, const float* k, const float* v, const float* decay, float* out,
                                       int batch, int heads, int kdim, int vdim, int l, int block_kdim,
                                       void* workspace, size_t workspace_bytes, void* stream) {{
  if (!rec_shape_ok(batch, heads, kdim, vdim, l, block_kdim)) return AAT_ERR_SHAPE;
  if (workspace == nullptr || workspace_bytes < total_workspace_bytes(batch, heads, vdim, l, block_kdim)) return AAT_ERR_WORKSPACE;
  return (int)launch(q, k, v, decay, out, batch, heads, kdim, vdim, l, block_kdim, static_cast<char*>(workspace),
                     static_cast<hipStream_t>(stream));
}}

extern "C" float retnet_recurrent_profile(const float* q, const float* k, const float* v, const float* decay, float* out,
                                          int batch, int heads, int kdim, int vdim, int l, int block_kdim,
                                          void* workspace, size_t workspace_bytes, void* stream) {{
  if (!rec_shape_ok(batch, heads, kdim, vdim, l, block_kdim)) return -1.f;
  if (workspace == nullptr || workspace_bytes < total_workspace_bytes(batch, heads, vdim, l, block_kdim)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&]() {{
    return launch(q, k, v, decay, out, batch, heads, kdim, vdim, l, block_kdim, static_cast<char*>(workspace), s);
  }});
}}

// No hipMalloc, no hipFree, no workspace argument: the decay factors go into `scratch`.  The factor kernel
// writes every byte of every record the scan reads, so nothing of an earlier call survives into this one
// and nothing has to be cleared.
extern "C" int retnet_recurrent_fwd_noalloc(const float* q, const float* k, const float* v, const float* decay, float* out,
                                            int batch, int heads, int kdim, int vdim, int l, int block_kdim, void* stream) {{
  if (!rec_shape_ok(batch, heads, kdim, vdim, l, block_kdim)) return AAT_ERR_SHAPE;
  if (block_kdim > 128 || (size_t)heads * (size_t)(l / 32) > (size_t)AAT_RECURRENT_NOALLOC_MAX_RECORDS) return AAT_ERR_LIMIT;
  char* ws = nullptr;
  const hipError_t e = scratch_of_current_device(&ws);
  if (e != hipSuccess) return (int)e;
  return (int)launch(q, k, v, decay, out, batch, heads, kdim, vdim, l, block_kdim, ws, static_cast<hipStream_t>(stream));
}}

// The reference's own entry point: same name, same arguments, no status, null stream.  An unsupported
// shape or a failed allocation is reported on stderr and leaves `out` untouched.
extern "C" void retnet_recurrent_fwd(void* d_q, void* d_k, void* d_v, void* d_decay, void* d_out, int batch, int heads,
                                     int kdim, int vdim, int l, int block_kdim) {{
  if (!rec_shape_ok(batch, heads, kdim, vdim, l, block_kdim)) {{
    std::fprintf(stderr, "retnet_recurrent_fwd: unsupported shape (l %% 32 == 0, block_kdim a multiple of 64 up to 256, vdim %% 64 == 0)\n");
    return;
  }}
  // Up to 128 key dims and AAT_RECURRENT_NOALLOC_MAX_RECORDS (head, chunk) pairs -- the reference benchmark's shape
  // among them -- the decay factors fit the array this library carries in its code object and nothing is allocated,
  // as the reference's own entry point allocates nothing; beyond that a per-device buffer is allocated once and kept.
  char* ws = nullptr;
  if (block_kdim <= 128 && (size_t)heads * (size_t)(l / 32) <= (size_t)AAT_RECURRENT_NOALLOC_MAX_RECORDS) {{
    const hipError_t es = scratch_of_current_device(&ws);
    if (es != hipSuccess) {{
      std::fprintf(stderr, "retnet_recurrent_fwd: %s\n", hipGetErrorString(es));
      return;
    }}
  }} else {{
    const size_t need = total_workspace_bytes(batch, heads, vdim, l, block_kdim);
    ws = cached_workspace(need);
    if (ws == nullptr) {{
      std::fprintf(stderr, "retnet_recurrent_fwd: cannot allocate %zu bytes of workspace\n", need);
      return;
    }}
  }}
  const hipError_t e = launch(static_cast<const float*>(d_q), static_cast<const float*>(d_k), static_cast<const float*>(d_v),
                              static_cast<const float*>(d_decay), static_cast<float*>(d_out), batch, heads, kdim, vdim, l,
                              block_kdim, ws, nullptr);
  if (e != hipSuccess) std::fprintf(stderr, "retnet_recurrent_fwd: %s\n", hipGetErrorString(e));
}}
"""

profile_code = kernel_code
