"""Source text of the per-configuration wrapper for the RetNet backward passes
(same role as reference csrc/kernels/retnet/bwd/profile_code.py:1-119).

One library launches three passes of the chained-contraction kernel (dV, dK, dQ); ``Br`` is the number
of block-resident rows and ``Bc`` the number of streamed rows per step of every pass.  ``dqaccum`` is
accepted for ABI compatibility and never touched: dQ is produced directly, without atomics.
"""

global_vars = r"""
#define AAT_OP_RET_BWD 1
#include "aat_kernel_abi.h"
#include "kernels/retnet/bwd/bwd_chain.h"
#include "kernels/utils/host_launch.h"

namespace {{
constexpr int Br = {Br};                 // block-resident rows of every pass
constexpr int Bc = {Bc};                 // streamed rows per step of every pass
constexpr int Kd = {Kd};
constexpr int D = {D};
constexpr int Nthreads = {Nthreads};
constexpr int num_stages_qk = {num_stages_qk};   // LDS buffers of the first-contraction stream (+ mask)
constexpr int num_stages_dv = {num_stages_dv};   // LDS buffers of the second-contraction stream
constexpr int waves_per_eu = {waves_per_eu};
// dV columns per block: the whole row when the accumulators fit the 256 accumulation registers that one
// wave per SIMD has to itself, else 256-column slices over grid.y (each repeats the first contraction).
constexpr int RTv = Br / (Nthreads / 64) / 32;
constexpr int DVB = (waves_per_eu == 1 && RTv * D <= 512) ? D : (D > 256 ? 256 : D);
constexpr int DKB = Kd;

using aat::BwdPass;
using TV = aat::RetBwdChain<Kd, D, DVB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col>;
using TK = aat::RetBwdChain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col>;
using TQ = aat::RetBwdChain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Row>;
const auto kernel_dv = &aat::ret_bwd_chain<Kd, D, DVB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col, waves_per_eu>;
const auto kernel_dk = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col, waves_per_eu>;
const auto kernel_dq = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Row, waves_per_eu>;
const auto decay_dv = &aat::ret_bwd_chain<Kd, D, DVB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col, waves_per_eu, true>;
const auto decay_dk = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col, waves_per_eu, true>;
const auto decay_dq = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Row, waves_per_eu, true>;

bool bwd_shape_ok(int B, int H, int Seq_q, int Seq_k) {{
  // every sequence length plays both roles (resident rows in one pass, streamed rows in another)
  return aat::shape_ok(B, H, Seq_q, Seq_k, Br, Br) && aat::shape_ok(B, H, Seq_q, Seq_k, Bc, Bc);
}}

hipError_t launch(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r, aat_half* dq,
                  aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, int mask_mode, void* workspace,
                  hipStream_t stream) {{
  static const hipError_t ok1 = aat::allow_lds(kernel_dv, TV::kSmemBytes);
  static const hipError_t ok2 = aat::allow_lds(kernel_dk, TK::kSmemBytes);
  static const hipError_t ok3 = aat::allow_lds(kernel_dq, TQ::kSmemBytes);
  if (ok1 != hipSuccess) return ok1;
  if (ok2 != hipSuccess) return ok2;
  if (ok3 != hipSuccess) return ok3;
  using H16 = aat::half_t;
  const H16 *Q = reinterpret_cast<const H16*>(q), *K = reinterpret_cast<const H16*>(k), *V = reinterpret_cast<const H16*>(v),
            *M = reinterpret_cast<const H16*>(mask), *G = reinterpret_cast<const H16*>(dO);
  aat::MaskWalk walk;
  const hipError_t scanned = aat::prepare_mask_walk(mask_mode, M, H, Seq_q, Seq_k, workspace, stream, &walk);
  if (scanned != hipSuccess) return scanned;
  const int causal = walk.causal;
  kernel_dv<<<dim3(B * H * (Seq_k / Br), D / DVB), dim3(Nthreads), TV::kSmemBytes, stream>>>(
      K, Q, G, M, r, reinterpret_cast<H16*>(dv), H, Seq_k, Seq_q, causal, nullptr, walk.extents);
  kernel_dk<<<dim3(B * H * (Seq_k / Br), Kd / DKB), dim3(Nthreads), TK::kSmemBytes, stream>>>(
      V, G, Q, M, r, reinterpret_cast<H16*>(dk), H, Seq_k, Seq_q, causal, nullptr, walk.extents);
  kernel_dq<<<dim3(B * H * (Seq_q / Br), Kd / DKB), dim3(Nthreads), TQ::kSmemBytes, stream>>>(
      G, V, K, M, r, reinterpret_cast<H16*>(dq), H, Seq_k, Seq_q, causal, nullptr, walk.extents);
  return hipGetLastError();
}}
// Decay-mask variant: the mask is gamma_h^(q + Seq_k - Seq_q - kv) below the diagonal, zero above it.
hipError_t launch_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* dO, float* r,
                        aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, hipStream_t stream) {{
  static const hipError_t ok1 = aat::allow_lds(decay_dv, TV::kSmemBytes);
  static const hipError_t ok2 = aat::allow_lds(decay_dk, TK::kSmemBytes);
  static const hipError_t ok3 = aat::allow_lds(decay_dq, TQ::kSmemBytes);
  if (ok1 != hipSuccess) return ok1;
  if (ok2 != hipSuccess) return ok2;
  if (ok3 != hipSuccess) return ok3;
  using H16 = aat::half_t;
  const H16 *Q = reinterpret_cast<const H16*>(q), *K = reinterpret_cast<const H16*>(k), *V = reinterpret_cast<const H16*>(v),
            *G = reinterpret_cast<const H16*>(dO);
  decay_dv<<<dim3(B * H * (Seq_k / Br), D / DVB), dim3(Nthreads), TV::kSmemBytes, stream>>>(
      K, Q, G, nullptr, r, reinterpret_cast<H16*>(dv), H, Seq_k, Seq_q, 1, log2_gamma, nullptr);
  decay_dk<<<dim3(B * H * (Seq_k / Br), Kd / DKB), dim3(Nthreads), TK::kSmemBytes, stream>>>(
      V, G, Q, nullptr, r, reinterpret_cast<H16*>(dk), H, Seq_k, Seq_q, 1, log2_gamma, nullptr);
  decay_dq<<<dim3(B * H * (Seq_q / Br), Kd / DKB), dim3(Nthreads), TQ::kSmemBytes, stream>>>(
      G, V, K, nullptr, r, reinterpret_cast<H16*>(dq), H, Seq_k, Seq_q, 1, log2_gamma, nullptr);
  return hipGetLastError();
}}
}}  // namespace

extern "C" int abi_version(void) {{ return AAT_ABI_VERSION; }}
extern "C" const char* config_string(void) {{ return "{config_name}"; }}
// Needed for the scanning mask modes only (AAT_MASK_SCAN / AAT_MASK_SCANNED); the same layout as the forward's.
extern "C" size_t workspace_size(int, int H, int Seq_q, int Seq_k) {{
  return H > 0 && Seq_q > 0 && Seq_k > 0 ? aat::mask_extent_bytes(H, Seq_q, Seq_k) : 0;
}}
static_assert(AAT_MASK_DENSE == aat::kMaskDense && AAT_MASK_CAUSAL == aat::kMaskCausal && AAT_MASK_SCAN == aat::kMaskScan &&
              AAT_MASK_SCANNED == aat::kMaskScanned, "mask modes of the header and of the kernels");
"""

profile_func = r"""
extern "C" float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r, aat_half* dq,
                            aat_half* dk, aat_half* dv, float*, int B, int H, int Seq_q, int Seq_k, int causal,
                            void* workspace, size_t workspace_bytes, void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k)) return -1.f;
  if (!aat::mask_mode_ok(causal, workspace, workspace_bytes, H, Seq_q, Seq_k)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{ return launch(q, k, v, mask, dO, r, dq, dk, dv, B, H, Seq_q, Seq_k, causal, workspace, s); }});
}}
extern "C" float profile(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r, aat_half* dq,
                         aat_half* dk, aat_half* dv, float* dqaccum, int B, int H, int Seq_q, int Seq_k) {{
  return profile_ex(q, k, v, mask, dO, r, dq, dk, dv, dqaccum, B, H, Seq_q, Seq_k, 0, nullptr, 0, nullptr);
}}
"""

kernel_entry = r"""
extern "C" int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r,
                               aat_half* dq, aat_half* dk, aat_half* dv, float*, int B, int H, int Seq_q, int Seq_k,
                               int causal, void* workspace, size_t workspace_bytes, void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k) || causal < 0 || causal > AAT_MASK_SCANNED) return AAT_ERR_SHAPE;
  if (!aat::mask_mode_ok(causal, workspace, workspace_bytes, H, Seq_q, Seq_k)) return AAT_ERR_WORKSPACE;
  return (int)launch(q, k, v, mask, dO, r, dq, dk, dv, B, H, Seq_q, Seq_k, causal, workspace, static_cast<hipStream_t>(stream));
}}
extern "C" int kernel_entry(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r, aat_half* dq,
                            aat_half* dk, aat_half* dv, float* dqaccum, int B, int H, int Seq_k, int Seq_q) {{
  return kernel_entry_ex(q, k, v, mask, dO, r, dq, dk, dv, dqaccum, B, H, Seq_q, Seq_k, 0, nullptr, 0, nullptr);
}}
"""

decay_entry = r"""
extern "C" float profile_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* dO, float* r,
                               aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, void*, size_t,
                               void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{ return launch_decay(q, k, v, log2_gamma, dO, r, dq, dk, dv, B, H, Seq_q, Seq_k, s); }});
}}
extern "C" int kernel_entry_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* dO, float* r,
                                  aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, void*,
                                  size_t, void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k)) return AAT_ERR_SHAPE;
  return (int)launch_decay(q, k, v, log2_gamma, dO, r, dq, dk, dv, B, H, Seq_q, Seq_k, static_cast<hipStream_t>(stream));
}}
"""

profile_code = global_vars + profile_func + kernel_entry + decay_entry
kernel_code = profile_code
