"""Source text of the per-configuration wrapper for the LDS-fused attention forward kernel.

``str.format_map(config.__dict__)`` fills the ``{Br}``-style fields; the result is one ``.hip`` file
that instantiates the kernel template for that configuration and exports the C ABI declared in
include/aat_kernel_abi.h.  Same role as reference csrc/kernels/attention/smemfuse/profile_code.py:1-93.
"""

global_vars = r"""
#define AAT_OP_ATTN 1
#include "aat_kernel_abi.h"
#include "kernels/attention/smemfuse/smemfuse.h"
#include "kernels/utils/host_launch.h"

namespace {{
constexpr int Br = {Br};
constexpr int Bc = {Bc};
constexpr int Kd = {Kd};
constexpr int D = {D};
constexpr int Nthreads = {Nthreads};
constexpr int num_stages_qk = {num_stages_qk};   // LDS buffers for the K tile
constexpr int num_stages_v = {num_stages_v};     // LDS buffers for the V tile
constexpr int waves_per_eu = {waves_per_eu};
constexpr int warps_mma1_N = {warps_mma1_n};    // waves along kv in S^T = K Q^T
constexpr int warps_mma_N = {warps_mma_n};      // waves along d in O^T = V^T P^T
constexpr float kReferenceScale = 0.125f;        // what the reference kernels hard-code

using Traits = aat::AttnFwdSmemfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, warps_mma1_N, warps_mma_N>;
constexpr int shared_mem = Traits::kSmemBytes;
const auto kernel = &aat::flashattn_fwd_smemfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, warps_mma1_N, warps_mma_N, waves_per_eu, false>;
const auto kernel_causal = &aat::flashattn_fwd_smemfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, warps_mma1_N, warps_mma_N, waves_per_eu, true>;

hipError_t launch(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k,
                  float softmax_scale, int causal, hipStream_t stream, float* lse = nullptr) {{
  static const hipError_t lds_ok = aat::allow_lds(kernel, shared_mem);
  static const hipError_t lds_ok_causal = aat::allow_lds(kernel_causal, shared_mem);
  if (lds_ok != hipSuccess) return lds_ok;
  if (lds_ok_causal != hipSuccess) return lds_ok_causal;
  (causal ? kernel_causal : kernel)<<<dim3(B * H * (Seq_q / Br)), dim3(Nthreads), shared_mem, stream>>>(
      reinterpret_cast<const aat::half_t*>(q), reinterpret_cast<const aat::half_t*>(k),
      reinterpret_cast<const aat::half_t*>(v), reinterpret_cast<aat::half_t*>(o), lse, H, Seq_k, Seq_q,
      softmax_scale);
  return hipGetLastError();
}}
}}  // namespace

extern "C" int abi_version(void) {{ return AAT_ABI_VERSION; }}
extern "C" const char* config_string(void) {{ return "{config_name}"; }}
extern "C" size_t workspace_size(int, int, int, int) {{ return 0; }}
"""

profile_func = r"""
extern "C" float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k,
                            float softmax_scale, int causal, void*, size_t, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{ return launch(q, k, v, o, B, H, Seq_q, Seq_k, softmax_scale, causal, s); }});
}}
extern "C" float profile(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k) {{
  return profile_ex(q, k, v, o, B, H, Seq_q, Seq_k, kReferenceScale, 0, nullptr, 0, nullptr);
}}
"""

kernel_entry = r"""
extern "C" int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k,
                               float softmax_scale, int causal, void*, size_t, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return AAT_ERR_SHAPE;
  return (int)launch(q, k, v, o, B, H, Seq_q, Seq_k, softmax_scale, causal, static_cast<hipStream_t>(stream));
}}
extern "C" int kernel_entry(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_k, int Seq_q) {{
  return kernel_entry_ex(q, k, v, o, B, H, Seq_q, Seq_k, kReferenceScale, 0, nullptr, 0, nullptr);
}}
extern "C" int kernel_entry_lse(aat_half* q, aat_half* k, aat_half* v, aat_half* o, float* lse, int B, int H, int Seq_q,
                                int Seq_k, float softmax_scale, int causal, void*, size_t, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return AAT_ERR_SHAPE;
  return (int)launch(q, k, v, o, B, H, Seq_q, Seq_k, softmax_scale, causal, static_cast<hipStream_t>(stream), lse);
}}
"""

# One library carries both halves of the ABI, so tuning and running share a single compile.
profile_code = global_vars + profile_func + kernel_entry
kernel_code = profile_code
