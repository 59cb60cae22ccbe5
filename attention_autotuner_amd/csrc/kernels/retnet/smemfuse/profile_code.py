"""Source text of the per-configuration wrapper for the LDS-fused RetNet forward kernel
(same role as reference csrc/kernels/retnet/smemfuse/profile_code.py:1-100)."""

global_vars = r"""
#define AAT_OP_RET 1
#include "aat_kernel_abi.h"
#include "kernels/retnet/smemfuse/smemfuse.h"
#include "kernels/utils/host_launch.h"

namespace {{
constexpr int Br = {Br};
constexpr int Bc = {Bc};
constexpr int Kd = {Kd};
constexpr int D = {D};
constexpr int Nthreads = {Nthreads};
constexpr int num_stages_qk = {num_stages_qk};     // LDS buffers for the K tile
constexpr int num_stages_mask = {num_stages_mask}; // LDS buffers for the mask tile (fetched with K)
constexpr int num_stages_v = {num_stages_v};       // LDS buffers for the V tile
constexpr int waves_per_eu = {waves_per_eu};
constexpr int warps_mma1_N = {warps_mma1_n};      // waves along kv in S^T = K Q^T
constexpr int warps_mma_N = {warps_mma_n};        // waves along d in O^T = V^T P^T
constexpr int stages_mask = num_stages_mask < num_stages_qk ? num_stages_qk : num_stages_mask;

using Traits = aat::RetFwdSmemfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, stages_mask, warps_mma1_N, warps_mma_N>;
constexpr int shared_mem = Traits::kSmemBytes;
const auto kernel = &aat::ret_fwd_smemfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, stages_mask, warps_mma1_N, warps_mma_N, waves_per_eu>;
const auto kernel_decay = &aat::ret_fwd_smemfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, stages_mask, warps_mma1_N, warps_mma_N, waves_per_eu, true>;

hipError_t launch(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r, int B, int H,
                  int Seq_q, int Seq_k, int mask_mode, void* workspace, hipStream_t stream) {{
  static const hipError_t lds_ok = aat::allow_lds(kernel, shared_mem);
  if (lds_ok != hipSuccess) return lds_ok;
  aat::MaskWalk walk;
  const hipError_t scanned = aat::prepare_mask_walk(mask_mode, reinterpret_cast<const aat::half_t*>(mask), H, Seq_q, Seq_k,
                                                    workspace, stream, &walk);
  if (scanned != hipSuccess) return scanned;
  kernel<<<dim3(B * H * (Seq_q / Br)), dim3(Nthreads), shared_mem, stream>>>(
      reinterpret_cast<const aat::half_t*>(q), reinterpret_cast<const aat::half_t*>(k),
      reinterpret_cast<const aat::half_t*>(v), reinterpret_cast<const aat::half_t*>(mask),
      reinterpret_cast<aat::half_t*>(o), r, H, Seq_k, Seq_q, walk.causal, nullptr, walk.extents);
  return hipGetLastError();
}}
// Decay-mask variant: the mask is gamma_h^(q + Seq_k - Seq_q - kv) below the diagonal, zero above it.
hipError_t launch_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* o, float* r, int B,
                        int H, int Seq_q, int Seq_k, hipStream_t stream) {{
  static const hipError_t lds_ok = aat::allow_lds(kernel_decay, shared_mem);
  if (lds_ok != hipSuccess) return lds_ok;
  kernel_decay<<<dim3(B * H * (Seq_q / Br)), dim3(Nthreads), shared_mem, stream>>>(
      reinterpret_cast<const aat::half_t*>(q), reinterpret_cast<const aat::half_t*>(k),
      reinterpret_cast<const aat::half_t*>(v), nullptr, reinterpret_cast<aat::half_t*>(o), r, H, Seq_k, Seq_q, 1,
      log2_gamma, nullptr);
  return hipGetLastError();
}}
}}  // namespace

extern "C" int abi_version(void) {{ return AAT_ABI_VERSION; }}
extern "C" const char* config_string(void) {{ return "{config_name}"; }}
// Needed for the scanning mask modes only (AAT_MASK_SCAN / AAT_MASK_SCANNED).
extern "C" size_t workspace_size(int, int H, int Seq_q, int Seq_k) {{
  return H > 0 && Seq_q > 0 && Seq_k > 0 ? aat::mask_extent_bytes(H, Seq_q, Seq_k) : 0;
}}
static_assert(AAT_MASK_DENSE == aat::kMaskDense && AAT_MASK_CAUSAL == aat::kMaskCausal && AAT_MASK_SCAN == aat::kMaskScan &&
              AAT_MASK_SCANNED == aat::kMaskScanned, "mask modes of the header and of the kernels");
"""

profile_func = r"""
extern "C" float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r, int B, int H,
                            int Seq_q, int Seq_k, int causal, void* workspace, size_t workspace_bytes, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return -1.f;
  if (!aat::mask_mode_ok(causal, workspace, workspace_bytes, H, Seq_q, Seq_k)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{ return launch(q, k, v, mask, o, r, B, H, Seq_q, Seq_k, causal, workspace, s); }});
}}
extern "C" float profile(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r, int B, int H,
                         int Seq_q, int Seq_k) {{
  return profile_ex(q, k, v, mask, o, r, B, H, Seq_q, Seq_k, 0, nullptr, 0, nullptr);
}}
"""

kernel_entry = r"""
extern "C" int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r, int B, int H,
                               int Seq_q, int Seq_k, int causal, void* workspace, size_t workspace_bytes, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc) || causal < 0 || causal > AAT_MASK_SCANNED) return AAT_ERR_SHAPE;
  if (!aat::mask_mode_ok(causal, workspace, workspace_bytes, H, Seq_q, Seq_k)) return AAT_ERR_WORKSPACE;
  return (int)launch(q, k, v, mask, o, r, B, H, Seq_q, Seq_k, causal, workspace, static_cast<hipStream_t>(stream));
}}
extern "C" int kernel_entry(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* o, float* r, int B, int H,
                            int Seq_k, int Seq_q) {{
  return kernel_entry_ex(q, k, v, mask, o, r, B, H, Seq_q, Seq_k, 0, nullptr, 0, nullptr);
}}
"""

decay_entry = r"""
extern "C" float profile_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* o, float* r,
                               int B, int H, int Seq_q, int Seq_k, void*, size_t, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{ return launch_decay(q, k, v, log2_gamma, o, r, B, H, Seq_q, Seq_k, s); }});
}}
extern "C" int kernel_entry_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* o, float* r,
                                  int B, int H, int Seq_q, int Seq_k, void*, size_t, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return AAT_ERR_SHAPE;
  return (int)launch_decay(q, k, v, log2_gamma, o, r, B, H, Seq_q, Seq_k, static_cast<hipStream_t>(stream));
}}
"""

profile_code = global_vars + profile_func + kernel_entry + decay_entry
kernel_code = profile_code
