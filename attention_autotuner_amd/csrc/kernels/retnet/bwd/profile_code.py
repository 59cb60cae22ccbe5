"""Source text of the per-configuration wrapper for the RetNet backward passes
(same role as reference csrc/kernels/retnet/bwd/profile_code.py:1-119).

One library launches three passes of the chained-contraction kernel (dV, dK, dQ); ``Br`` is the number
of block-resident rows and ``Bc`` the number of streamed rows per step of every pass.  ``dqaccum`` is
accepted for ABI compatibility and never touched: dQ is produced directly, without atomics.

With ``ds_rows`` set the dQ pass runs before dK and stores its dS tiles in the workspace (behind the mask scan's
ranges), and dK comes from the kernel that reads them back (dk_from_ds.h); ``workspace_size`` says how much room that
takes, and without it the library runs the chained dK pass.
"""

global_vars = r"""
#define AAT_OP_RET_BWD 1
#include "aat_kernel_abi.h"
#include "kernels/retnet/bwd/bwd_chain.h"
#include "kernels/retnet/bwd/dk_from_ds.h"
#include "kernels/utils/host_launch.h"

namespace {{
constexpr int Br = {Br};                 // block-resident rows of every pass
constexpr int Bc = {Bc};                 // streamed rows per step of every pass
constexpr int Kd = {Kd};
constexpr int D = {D};
constexpr int Nthreads = {Nthreads};
constexpr int num_stages_qk = {num_stages_qk};   // LDS buffers of the first-contraction stream (+ mask)
constexpr int num_stages_dv = {num_stages_dv};   // LDS buffers of the second-contraction stream
// the same two counts for the passes that contract over d_v first (dQ, and dK when it is a chained pass): their streamed
// tiles are d_v wide, twice the dV pass's at d_v = 2 d_qk, so they often cannot afford what the dV pass can
constexpr int num_stages_ds = {num_stages_ds};
constexpr int num_stages_dq = {num_stages_dq};
constexpr int waves_per_eu = {waves_per_eu};
constexpr int ds_rows = {ds_rows};               // 0, or kv rows per block of the dK kernel that reads a stored dS
constexpr bool kStoredDs = ds_rows != 0;
constexpr int kDkRows = kStoredDs ? ds_rows : 128, kDkTile = 64, kDkStages = 2, kDkWaves = 2;
// dV columns per block: the whole row when the accumulators fit the 256 accumulation registers that one
// wave per SIMD has to itself, else 256-column slices over grid.y (each repeats the first contraction).
constexpr int RTv = Br / (Nthreads / 64) / 32;
constexpr int DVB = (waves_per_eu == 1 && RTv * D <= 512) ? D : (D > 256 ? 256 : D);
constexpr int DKB = Kd;

using aat::BwdPass;
using TV = aat::RetBwdChain<Kd, D, DVB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col>;
using TK = aat::RetBwdChain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_ds, num_stages_dq, BwdPass::Col>;
using TQ = aat::RetBwdChain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_ds, num_stages_dq, BwdPass::Row>;
const auto kernel_dv = &aat::ret_bwd_chain<Kd, D, DVB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col, waves_per_eu>;
const auto kernel_dk = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_ds, num_stages_dq, BwdPass::Col, waves_per_eu>;
const auto kernel_dq = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_ds, num_stages_dq, BwdPass::Row, waves_per_eu>;
const auto decay_dv = &aat::ret_bwd_chain<Kd, D, DVB, Br, Bc, Nthreads, num_stages_qk, num_stages_dv, BwdPass::Col, waves_per_eu, true>;
const auto decay_dk = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_ds, num_stages_dq, BwdPass::Col, waves_per_eu, true>;
const auto decay_dq = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_ds, num_stages_dq, BwdPass::Row, waves_per_eu, true>;
// stored dS: the row pass that writes it (the plain one again in a library without it), the dK kernel that reads it
using TKD = aat::RetBwdDk<Kd, kDkRows, kDkTile, kDkRows * 2, kDkStages>;
const auto kernel_dq_ds = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_ds, num_stages_dq, BwdPass::Row, waves_per_eu, false, kStoredDs>;
const auto decay_dq_ds = &aat::ret_bwd_chain<D, Kd, DKB, Br, Bc, Nthreads, num_stages_ds, num_stages_dq, BwdPass::Row, waves_per_eu, true, kStoredDs>;
const auto kernel_dk_ds = &aat::ret_bwd_dk_from_ds<Kd, kDkRows, kDkTile, kDkRows * 2, kDkStages, kDkWaves>;
static_assert(!kStoredDs || Br % kDkTile == 0, "a query tile of the dK kernel lies inside one block of the row pass");

bool bwd_shape_ok(int B, int H, int Seq_q, int Seq_k) {{
  // every sequence length plays both roles (resident rows in one pass, streamed rows in another)
  return aat::shape_ok(B, H, Seq_q, Seq_k, Br, Br) && aat::shape_ok(B, H, Seq_q, Seq_k, Bc, Bc);
}}
// whether this library stores dS for the problem: it is built for it and the lengths fit the dK kernel's tiles
bool stores_ds(int B, int H, int Seq_q, int Seq_k) {{ return kStoredDs && aat::shape_ok(B, H, Seq_q, Seq_k, kDkTile, kDkRows); }}

// Workspace: the mask scan's ranges (as the forward lays them out), then, with a stored dS, B*H*Seq_q*Seq_k fp16.
size_t ds_offset(int H, int Seq_q, int Seq_k) {{ return aat::mask_extent_bytes(H, Seq_q, Seq_k); }}
size_t ws_bytes_needed(int B, int H, int Seq_q, int Seq_k) {{
  const size_t scan = aat::mask_extent_bytes(H, Seq_q, Seq_k);
  return stores_ds(B, H, Seq_q, Seq_k) ? scan + (size_t)B * H * Seq_q * Seq_k * sizeof(aat::half_t) : scan;
}}
// The scanning modes need the ranges.  dS is stored when the workspace has its room too; without it (the
// reference-signature entry points have no workspace to give) dK comes from the chained pass that evaluates dS again.
bool workspace_ok(int mode, const void* workspace, size_t workspace_bytes, int H, int Seq_q, int Seq_k) {{
  return aat::mask_mode_ok(mode, workspace, workspace_bytes, H, Seq_q, Seq_k);
}}
bool room_for_ds(const void* workspace, size_t workspace_bytes, int B, int H, int Seq_q, int Seq_k) {{
  return stores_ds(B, H, Seq_q, Seq_k) && workspace != nullptr && workspace_bytes >= ws_bytes_needed(B, H, Seq_q, Seq_k);
}}

hipError_t launch(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r, aat_half* dq,
                  aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, int mask_mode, void* workspace,
                  size_t workspace_bytes, hipStream_t stream) {{
  static const hipError_t ok1 = aat::allow_lds(kernel_dv, TV::kSmemBytes);
  static const hipError_t ok2 = aat::allow_lds(kernel_dk, TK::kSmemBytes);
  static const hipError_t ok3 = aat::allow_lds(kernel_dq, TQ::kSmemBytes);
  static const hipError_t ok4 = kStoredDs ? aat::allow_lds(kernel_dk_ds, TKD::kSmemBytes) : hipSuccess;
  static const hipError_t ok5 = kStoredDs ? aat::allow_lds(kernel_dq_ds, TQ::kSmemBytesDsOut) : hipSuccess;
  for (hipError_t e : {{ok1, ok2, ok3, ok4, ok5}})
    if (e != hipSuccess) return e;
  using H16 = aat::half_t;
  const H16 *Q = reinterpret_cast<const H16*>(q), *K = reinterpret_cast<const H16*>(k), *V = reinterpret_cast<const H16*>(v),
            *M = reinterpret_cast<const H16*>(mask), *G = reinterpret_cast<const H16*>(dO);
  aat::MaskWalk walk;
  const hipError_t scanned = aat::prepare_mask_walk(mask_mode, M, H, Seq_q, Seq_k, workspace, stream, &walk);
  if (scanned != hipSuccess) return scanned;
  const int causal = walk.causal;
  kernel_dv<<<dim3(B * H * (Seq_k / Br), D / DVB), dim3(Nthreads), TV::kSmemBytes, stream>>>(
      K, Q, G, M, r, reinterpret_cast<H16*>(dv), H, Seq_k, Seq_q, causal, nullptr, walk.extents, nullptr);
  if (room_for_ds(workspace, workspace_bytes, B, H, Seq_q, Seq_k)) {{
    H16* ds = reinterpret_cast<H16*>(static_cast<char*>(workspace) + ds_offset(H, Seq_q, Seq_k));
    kernel_dq_ds<<<dim3(B * H * (Seq_q / Br), Kd / DKB), dim3(Nthreads), TQ::kSmemBytesDsOut, stream>>>(
        G, V, K, M, r, reinterpret_cast<H16*>(dq), H, Seq_k, Seq_q, causal, nullptr, walk.extents, ds);
    kernel_dk_ds<<<dim3(B * H * (Seq_k / kDkRows)), dim3(kDkRows * 2), TKD::kSmemBytes, stream>>>(
        Q, ds, reinterpret_cast<H16*>(dk), H, Seq_k, Seq_q, causal, walk.extents, Br, Bc);
  }} else {{
    kernel_dk<<<dim3(B * H * (Seq_k / Br), Kd / DKB), dim3(Nthreads), TK::kSmemBytes, stream>>>(
        V, G, Q, M, r, reinterpret_cast<H16*>(dk), H, Seq_k, Seq_q, causal, nullptr, walk.extents, nullptr);
    kernel_dq<<<dim3(B * H * (Seq_q / Br), Kd / DKB), dim3(Nthreads), TQ::kSmemBytes, stream>>>(
        G, V, K, M, r, reinterpret_cast<H16*>(dq), H, Seq_k, Seq_q, causal, nullptr, walk.extents, nullptr);
  }}
  return hipGetLastError();
}}
// Decay-mask variant: the mask is gamma_h^(q + Seq_k - Seq_q - kv) below the diagonal, zero above it.
hipError_t launch_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* dO, float* r,
                        aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, void* workspace,
                        size_t workspace_bytes, hipStream_t stream) {{
  static const hipError_t ok1 = aat::allow_lds(decay_dv, TV::kSmemBytes);
  static const hipError_t ok2 = aat::allow_lds(decay_dk, TK::kSmemBytes);
  static const hipError_t ok3 = aat::allow_lds(decay_dq, TQ::kSmemBytes);
  static const hipError_t ok4 = kStoredDs ? aat::allow_lds(kernel_dk_ds, TKD::kSmemBytes) : hipSuccess;
  static const hipError_t ok5 = kStoredDs ? aat::allow_lds(decay_dq_ds, TQ::kSmemBytesDsOut) : hipSuccess;
  for (hipError_t e : {{ok1, ok2, ok3, ok4, ok5}})
    if (e != hipSuccess) return e;
  using H16 = aat::half_t;
  const H16 *Q = reinterpret_cast<const H16*>(q), *K = reinterpret_cast<const H16*>(k), *V = reinterpret_cast<const H16*>(v),
            *G = reinterpret_cast<const H16*>(dO);
  decay_dv<<<dim3(B * H * (Seq_k / Br), D / DVB), dim3(Nthreads), TV::kSmemBytes, stream>>>(
      K, Q, G, nullptr, r, reinterpret_cast<H16*>(dv), H, Seq_k, Seq_q, 1, log2_gamma, nullptr, nullptr);
  if (room_for_ds(workspace, workspace_bytes, B, H, Seq_q, Seq_k)) {{
    H16* ds = reinterpret_cast<H16*>(static_cast<char*>(workspace) + ds_offset(H, Seq_q, Seq_k));
    decay_dq_ds<<<dim3(B * H * (Seq_q / Br), Kd / DKB), dim3(Nthreads), TQ::kSmemBytesDsOut, stream>>>(
        G, V, K, nullptr, r, reinterpret_cast<H16*>(dq), H, Seq_k, Seq_q, 1, log2_gamma, nullptr, ds);
    kernel_dk_ds<<<dim3(B * H * (Seq_k / kDkRows)), dim3(kDkRows * 2), TKD::kSmemBytes, stream>>>(
        Q, ds, reinterpret_cast<H16*>(dk), H, Seq_k, Seq_q, 1, nullptr, Br, Bc);
  }} else {{
    decay_dk<<<dim3(B * H * (Seq_k / Br), Kd / DKB), dim3(Nthreads), TK::kSmemBytes, stream>>>(
        V, G, Q, nullptr, r, reinterpret_cast<H16*>(dk), H, Seq_k, Seq_q, 1, log2_gamma, nullptr, nullptr);
    decay_dq<<<dim3(B * H * (Seq_q / Br), Kd / DKB), dim3(Nthreads), TQ::kSmemBytes, stream>>>(
        G, V, K, nullptr, r, reinterpret_cast<H16*>(dq), H, Seq_k, Seq_q, 1, log2_gamma, nullptr, nullptr);
  }}
  return hipGetLastError();
}}
}}  // namespace

extern "C" int abi_version(void) {{ return AAT_ABI_VERSION; }}
extern "C" const char* config_string(void) {{ return "{config_name}"; }}
// The ranges of the scanning mask modes (AAT_MASK_SCAN / AAT_MASK_SCANNED; the same layout as the forward's, so a scan
// the forward made can be handed over or copied to the head of a larger buffer) and, with a stored dS, its room (a
// smaller workspace is accepted: dK then comes from the chained pass).
extern "C" size_t workspace_size(int B, int H, int Seq_q, int Seq_k) {{
  return B > 0 && H > 0 && Seq_q > 0 && Seq_k > 0 ? ws_bytes_needed(B, H, Seq_q, Seq_k) : 0;
}}

static_assert(AAT_MASK_DENSE == aat::kMaskDense && AAT_MASK_CAUSAL == aat::kMaskCausal && AAT_MASK_SCAN == aat::kMaskScan &&
              AAT_MASK_SCANNED == aat::kMaskScanned, "mask modes of the header and of the kernels");
"""

profile_func = r"""
extern "C" float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r, aat_half* dq,
                            aat_half* dk, aat_half* dv, float*, int B, int H, int Seq_q, int Seq_k, int causal,
                            void* workspace, size_t workspace_bytes, void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k)) return -1.f;
  if (!workspace_ok(causal, workspace, workspace_bytes, H, Seq_q, Seq_k)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{ return launch(q, k, v, mask, dO, r, dq, dk, dv, B, H, Seq_q, Seq_k, causal, workspace, workspace_bytes, s); }});
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
  if (!workspace_ok(causal, workspace, workspace_bytes, H, Seq_q, Seq_k)) return AAT_ERR_WORKSPACE;
  return (int)launch(q, k, v, mask, dO, r, dq, dk, dv, B, H, Seq_q, Seq_k, causal, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}}
extern "C" int kernel_entry(aat_half* q, aat_half* k, aat_half* v, aat_half* mask, aat_half* dO, float* r, aat_half* dq,
                            aat_half* dk, aat_half* dv, float* dqaccum, int B, int H, int Seq_k, int Seq_q) {{
  return kernel_entry_ex(q, k, v, mask, dO, r, dq, dk, dv, dqaccum, B, H, Seq_q, Seq_k, 0, nullptr, 0, nullptr);
}}
"""

decay_entry = r"""
extern "C" float profile_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* dO, float* r,
                               aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k, void* workspace,
                               size_t workspace_bytes, void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k)) return -1.f;
  if (!workspace_ok(AAT_MASK_CAUSAL, workspace, workspace_bytes, H, Seq_q, Seq_k)) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{ return launch_decay(q, k, v, log2_gamma, dO, r, dq, dk, dv, B, H, Seq_q, Seq_k, workspace, workspace_bytes, s); }});
}}
extern "C" int kernel_entry_decay(aat_half* q, aat_half* k, aat_half* v, const float* log2_gamma, aat_half* dO, float* r,
                                  aat_half* dq, aat_half* dk, aat_half* dv, int B, int H, int Seq_q, int Seq_k,
                                  void* workspace, size_t workspace_bytes, void* stream) {{
  if (!bwd_shape_ok(B, H, Seq_q, Seq_k)) return AAT_ERR_SHAPE;
  if (!workspace_ok(AAT_MASK_CAUSAL, workspace, workspace_bytes, H, Seq_q, Seq_k)) return AAT_ERR_WORKSPACE;
  return (int)launch_decay(q, k, v, log2_gamma, dO, r, dq, dk, dv, B, H, Seq_q, Seq_k, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}}
"""

profile_code = global_vars + profile_func + kernel_entry + decay_entry
kernel_code = profile_code
