"""Source text of the per-configuration wrapper for the flash-attention backward.

The reference has no such wrapper (its attention operator's ``backward`` is empty, reference
python/ops/attention_interface.py:37-58); the layout follows its RetNet backward wrapper
(csrc/kernels/retnet/bwd/profile_code.py:1-119).  One library launches three kernels: the preparation
pass (delta = rowsum(dO * O), lse in base-2 units, both into the workspace), the column kernel (dV, dK)
and the row kernel (dQ); with ``col_split`` the column kernel runs twice, once per output.
"""

global_vars = r"""
#define AAT_OP_ATTN_BWD 1
#include "aat_kernel_abi.h"
#include "kernels/attention/bwd/bwd_chain.h"
#include "kernels/utils/host_launch.h"

namespace {{
constexpr int Br = {Br};                 // block-resident rows of both kernels
constexpr int Bc = {Bc};                 // streamed rows per step of the column kernel
constexpr int BcRow = {row_Bc};          // streamed rows per step of the row kernel
constexpr int Kd = {Kd};
constexpr int D = {D};
constexpr int Nthreads = {Nthreads};
constexpr int num_stages = {num_stages_qk};      // LDS buffers of the streamed tiles
constexpr int waves_per_eu = {waves_per_eu};
constexpr int row_waves_per_eu = {row_waves_per_eu};   // register budget of the row kernel (one output: fits 256 registers)
#define AAT_COL_SPLIT {col_split}                      // 1: one column kernel per output (dV, dK)
constexpr int dv_waves_per_eu = {dv_waves_per_eu};
constexpr int dk_waves_per_eu = {dk_waves_per_eu};

using aat::AttnBwdPass;
using TC = aat::AttnBwdChain<Kd, D, Br, Bc, Nthreads, num_stages, AttnBwdPass::Col>;
using TR = aat::AttnBwdChain<Kd, D, Br, BcRow, Nthreads, num_stages, AttnBwdPass::Row>;
#if AAT_COL_SPLIT
const auto kernel_dv = &aat::attn_bwd_chain<Kd, D, Br, Bc, Nthreads, num_stages, AttnBwdPass::Col, dv_waves_per_eu, 1>;
const auto kernel_dk = &aat::attn_bwd_chain<Kd, D, Br, Bc, Nthreads, num_stages, AttnBwdPass::Col, dk_waves_per_eu, 2>;
#else
const auto kernel_col = &aat::attn_bwd_chain<Kd, D, Br, Bc, Nthreads, num_stages, AttnBwdPass::Col, waves_per_eu>;
#endif
const auto kernel_row = &aat::attn_bwd_chain<Kd, D, Br, BcRow, Nthreads, num_stages, AttnBwdPass::Row, row_waves_per_eu>;

bool bwd_shape_ok(int B, int H, int Seq_q, int Seq_k) {{
  // every sequence length plays both roles (resident rows in one kernel, streamed rows in the other)
  return aat::shape_ok(B, H, Seq_q, Seq_k, Br, Br) && aat::shape_ok(B, H, Seq_q, Seq_k, Bc, BcRow);   // q rows stream through the column kernel, kv rows through the row kernel
}}
size_t stats_bytes(int B, int H, int Seq_q) {{ return (size_t)2 * B * H * Seq_q * sizeof(float); }}

hipError_t launch(aat_half* q, aat_half* k, aat_half* v, aat_half* o, aat_half* dO, float* lse, aat_half* dq,
                  aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, float softmax_scale, int causal,
                  void* workspace, hipStream_t stream) {{
#if AAT_COL_SPLIT
  static const hipError_t ok0 = aat::allow_lds(kernel_dv, TC::kSmemBytes);
  static const hipError_t ok1 = aat::allow_lds(kernel_dk, TC::kSmemBytes);
  if (ok0 != hipSuccess) return ok0;
#else
  static const hipError_t ok1 = aat::allow_lds(kernel_col, TC::kSmemBytes);
#endif
  static const hipError_t ok2 = aat::allow_lds(kernel_row, TR::kSmemBytes);
  if (ok1 != hipSuccess) return ok1;
  if (ok2 != hipSuccess) return ok2;
  using H16 = aat::half_t;
  const H16 *Q = reinterpret_cast<const H16*>(q), *K = reinterpret_cast<const H16*>(k), *V = reinterpret_cast<const H16*>(v),
            *O = reinterpret_cast<const H16*>(o), *G = reinterpret_cast<const H16*>(dO);
  const int rows = B * H * Seq_q;
  float* lse2 = static_cast<float*>(workspace);
  float* delta = lse2 + rows;
  constexpr int rows_per_block = aat::attn_bwd_prepare_rows_per_block<D>();
  aat::attn_bwd_prepare<D><<<dim3((rows + rows_per_block - 1) / rows_per_block), dim3(256), 0, stream>>>(O, G, lse, lse2, delta, rows);
  const float c2 = softmax_scale * 1.4426950408889634f;
#if AAT_COL_SPLIT
  kernel_dv<<<dim3(B * H * (Seq_k / Br)), dim3(Nthreads), TC::kSmemBytes, stream>>>(
      K, V, Q, G, lse2, delta, reinterpret_cast<H16*>(dv), nullptr, H, Seq_k, Seq_q, c2, softmax_scale, causal);
  kernel_dk<<<dim3(B * H * (Seq_k / Br)), dim3(Nthreads), TC::kSmemBytes, stream>>>(
      K, V, Q, G, lse2, delta, nullptr, reinterpret_cast<H16*>(dk), H, Seq_k, Seq_q, c2, softmax_scale, causal);
#else
  kernel_col<<<dim3(B * H * (Seq_k / Br)), dim3(Nthreads), TC::kSmemBytes, stream>>>(
      K, V, Q, G, lse2, delta, reinterpret_cast<H16*>(dv), reinterpret_cast<H16*>(dk), H, Seq_k, Seq_q, c2, softmax_scale, causal);
#endif
  kernel_row<<<dim3(B * H * (Seq_q / Br)), dim3(Nthreads), TR::kSmemBytes, stream>>>(
      Q, G, K, V, lse2, delta, nullptr, reinterpret_cast<H16*>(dq), H, Seq_k, Seq_q, c2, softmax_scale, causal);
  return hipGetLastError();
}}
}}  // namespace

extern "C" int abi_version(void) {{ return AAT_ABI_VERSION; }}
extern "C" const char* config_string(void) {{ return "{config_name}"; }}
extern "C" size_t workspace_size(int B, int H, int Seq_q, int) {{ return stats_bytes(B, H, Seq_q); }}
"""

profile_func = r"""
extern "C" float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, aat_half* dO, float* lse, aat_half* dq,
                            aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, float softmax_scale,
                            int causal, void* workspace, size_t workspace_bytes, void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k)) return -1.f;
  if (workspace == nullptr || workspace_bytes < stats_bytes(B, H, Seq_q)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{
    return launch(q, k, v, o, dO, lse, dq, dk, dv, B, H, Seq_q, Seq_k, softmax_scale, causal, workspace, s);
  }});
}}
"""

kernel_entry = r"""
extern "C" int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, aat_half* dO, float* lse, aat_half* dq,
                               aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, float softmax_scale,
                               int causal, void* workspace, size_t workspace_bytes, void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k)) return AAT_ERR_SHAPE;
  if (workspace == nullptr || workspace_bytes < stats_bytes(B, H, Seq_q)) return AAT_ERR_WORKSPACE;
  return (int)launch(q, k, v, o, dO, lse, dq, dk, dv, B, H, Seq_q, Seq_k, softmax_scale, causal, workspace,
                     static_cast<hipStream_t>(stream));
}}
"""

profile_code = global_vars + profile_func + kernel_entry
kernel_code = profile_code
