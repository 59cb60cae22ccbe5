"""Source text of the per-configuration wrapper for the register-fused attention forward kernel.

``str.format_map(config.__dict__)`` fills the ``{Br}``-style fields; the result is one ``.hip`` file
that instantiates the kernel template for that configuration and exports the C ABI declared in
include/aat_kernel_abi.h.  Same role as reference csrc/kernels/attention/regfuse/profile_code.py:1-79.
"""

global_vars = r"""
#define AAT_OP_ATTN 1
#include <atomic>
#include "aat_kernel_abi.h"
#include "kernels/attention/regfuse/regfuse.h"
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
constexpr int kv_splits = {kv_splits};           // > 1: the kv range is cut into that many parts (non-causal only)
constexpr bool sw_pipeline = {sw_pipeline};      // next tile's QK^T MFMAs interleaved with this tile's exponentials
constexpr int unit_rows = sw_pipeline ? Bc : {BlockKSmem2};   // plain schedule: kv rows per scores -> softmax -> PV unit inside a tile of Bc rows
constexpr float kReferenceScale = 0.125f;        // what the reference kernels hard-code

using Traits = aat::AttnFwdRegfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v>;
constexpr int shared_mem = Traits::kSmemBytes;
const auto kernel = &aat::flashattn_fwd_regfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, waves_per_eu, unit_rows, sw_pipeline, false>;
const auto kernel_causal = &aat::flashattn_fwd_regfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, waves_per_eu, unit_rows, sw_pipeline, true>;
const auto kernel_causal_paired = &aat::flashattn_fwd_regfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, waves_per_eu, unit_rows, sw_pipeline, true, false, false, true>;
const auto kernel_split = &aat::flashattn_fwd_regfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, waves_per_eu, unit_rows, sw_pipeline, false, true>;
constexpr int shared_mem_split = Traits::kSmemBytesSplit;

// Persistent variant (a block walks several row blocks, prefetching across them): exists for two K and two V
// buffers, the plain schedule and a tile shape that leaves room to stage the output beside the prefetched
// tiles; used for non-causal problems with an even number of kv tiles and more row blocks than the chip holds
// at once -- and with fewer than 2048 kv rows.  Measured with the Br=256 Bc=128 512-thread
// configuration under sustained load (300 launches back to back): +10 % at S=512 (B 16, H 32), +3 % at S=1024,
// +-0 at S=2048, -1.5 % at S=4096: what it removes is the 5.7 us a block spends per row block on start-up and
// drain, and on long rows the kernel runs at the chip's power limit, where idle time is not what bounds it.
constexpr int kPersistMaxKv = 1792;
using PersistTraits = Traits::Persist<waves_per_eu>;
constexpr int shared_mem_persist = PersistTraits::kSmemBytes;
template <bool OK> auto persistent_kernel() {{
  if constexpr (OK)
    return &aat::flashattn_fwd_regfuse<Kd, D, Br, Bc, Nthreads, num_stages_qk, num_stages_v, waves_per_eu, unit_rows, false, false, false, true>;
  else
    return static_cast<decltype(kernel)>(nullptr);
}}
const auto kernel_persist = persistent_kernel<PersistTraits::kOk && !sw_pipeline>();

// Blocks of the persistent kernel the current device holds at once (0: unknown, do not use it).
int resident_blocks() {{
  static std::atomic<int> cached[64];            // per device; threads that race here compute the same value
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int blocks = cached[dev].load(std::memory_order_relaxed);
  if (blocks == 0) {{
    int per_cu = 0, cus = 0;
    // The persistent kernel requests the next row block's Q fragments into live registers behind the compiler's back
    // and waits for them a tile later.  That is sound only while those registers stay registers: a build whose
    // allocator spilled anything (scratch bytes per lane != 0) may have parked a fragment in memory before it arrived.
    hipFuncAttributes attr;
    if (hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(kernel_persist)) != hipSuccess || attr.localSizeBytes != 0 ||
        aat::allow_lds(kernel_persist, shared_mem_persist) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kernel_persist), Nthreads, shared_mem_persist) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || per_cu <= 0 || cus <= 0)
      blocks = -1;
    else
      blocks = per_cu * cus;
    cached[dev].store(blocks, std::memory_order_relaxed);
  }}
  return blocks > 0 ? blocks : 0;
}}

// Whether `n` equal workgroups come out as whole rounds over the workgroups the chip holds at this configuration's
// occupancy (registers: waves_per_eu waves per SIMD; the LDS may allow fewer, which this does not look at).
bool pairs_fill_the_chip(int n) {{
  static std::atomic<int> cus_of[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
  int cus = cus_of[dev].load(std::memory_order_relaxed);
  if (cus == 0) {{
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = -1;
    cus_of[dev].store(cus, std::memory_order_relaxed);
  }}
  if (cus <= 0) return false;
  // a build of the paired kernel that keeps part of its working set in scratch memory (the second pass costs registers)
  // loses more than the pairing gains: the one-row-block-per-workgroup kernel stands in
  static const bool paired_spills = [] {{
    hipFuncAttributes attr;
    return hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(kernel_causal_paired)) != hipSuccess || attr.localSizeBytes != 0;
  }}();
  if (paired_spills) return false;
  const int per_cu = waves_per_eu * 4 * 64 / Nthreads > 0 ? waves_per_eu * 4 * 64 / Nthreads : 1;
  const int resident = cus * per_cu;
  return n % resident == 0 || n >= 8 * resident;
}}

size_t split_workspace_bytes(int B, int H, int Seq_q) {{
  return kv_splits > 1 ? (size_t)kv_splits * B * H * Seq_q * (D + 1) * sizeof(float) : 0;
}}
bool split_applies(int Seq_k, int causal) {{ return kv_splits > 1 && !causal && (Seq_k / Bc) % kv_splits == 0; }}

hipError_t launch(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k,
                  float softmax_scale, int causal, void* workspace, hipStream_t stream, float* lse = nullptr) {{
  if (split_applies(Seq_k, causal) && workspace != nullptr) {{
    static const hipError_t lds_ok_split = aat::allow_lds(kernel_split, shared_mem_split);
    if (lds_ok_split != hipSuccess) return lds_ok_split;
    const size_t rows = (size_t)B * H * Seq_q;
    float* part_o = static_cast<float*>(workspace);
    float* part_lse = part_o + (size_t)kv_splits * rows * D;
    kernel_split<<<dim3(B * H * (Seq_q / Br), kv_splits), dim3(Nthreads), shared_mem_split, stream>>>(
        reinterpret_cast<const aat::half_t*>(q), reinterpret_cast<const aat::half_t*>(k),
        reinterpret_cast<const aat::half_t*>(v), nullptr, nullptr, H, Seq_k, Seq_q, softmax_scale, part_o, part_lse, 0);
    const size_t threads = rows * (D / 8);
    aat::attn_split_merge<D><<<dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream>>>(
        part_o, part_lse, reinterpret_cast<aat::half_t*>(o), lse, (int)rows, kv_splits);
    return hipGetLastError();
  }}
  const int items = B * H * (Seq_q / Br);
  if (kernel_persist != nullptr && !causal && (Seq_k / Bc) % 2 == 0 && Seq_k <= kPersistMaxKv) {{
    const int resident = resident_blocks();
    if (resident > 0 && items > resident) {{
      kernel_persist<<<dim3(resident), dim3(Nthreads), shared_mem_persist, stream>>>(
          reinterpret_cast<const aat::half_t*>(q), reinterpret_cast<const aat::half_t*>(k),
          reinterpret_cast<const aat::half_t*>(v), reinterpret_cast<aat::half_t*>(o), lse, H, Seq_k, Seq_q,
          softmax_scale, nullptr, nullptr, items);
      return hipGetLastError();
    }}
  }}
  static const hipError_t lds_ok = aat::allow_lds(kernel, shared_mem);
  static const hipError_t lds_ok_causal = aat::allow_lds(kernel_causal, shared_mem);
  if (lds_ok != hipSuccess) return lds_ok;
  if (lds_ok_causal != hipSuccess) return lds_ok_causal;
  // causal, an even number of row blocks per head: half the grid, every workgroup walks a long and a short row block --
  // where those workgroups fill the chip a whole number of times (or many times over); a last round that is one third
  // full costs more than the equal lengths and the shared K/V stream gain
  const bool paired = causal && (Seq_q / Br) % 2 == 0 && pairs_fill_the_chip(items / 2);
  static const hipError_t lds_ok_paired = aat::allow_lds(kernel_causal_paired, shared_mem);
  if (lds_ok_paired != hipSuccess) return lds_ok_paired;
  (paired ? kernel_causal_paired : causal ? kernel_causal : kernel)<<<dim3(paired ? items / 2 : items), dim3(Nthreads), shared_mem, stream>>>(
      reinterpret_cast<const aat::half_t*>(q), reinterpret_cast<const aat::half_t*>(k),
      reinterpret_cast<const aat::half_t*>(v), reinterpret_cast<aat::half_t*>(o), lse, H, Seq_k, Seq_q,
      softmax_scale, nullptr, nullptr, 0);
  return hipGetLastError();
}}
}}  // namespace

extern "C" int abi_version(void) {{ return AAT_ABI_VERSION; }}
extern "C" const char* config_string(void) {{ return "{config_name}"; }}
extern "C" size_t workspace_size(int B, int H, int Seq_q, int) {{ return split_workspace_bytes(B, H, Seq_q); }}
"""

profile_func = r"""
extern "C" float profile_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k,
                            float softmax_scale, int causal, void* workspace, size_t workspace_bytes, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return -1.f;
  if (split_applies(Seq_k, causal) && (workspace == nullptr || workspace_bytes < split_workspace_bytes(B, H, Seq_q))) return -1.f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return aat::timed_mean_ms(s, [&] {{ return launch(q, k, v, o, B, H, Seq_q, Seq_k, softmax_scale, causal, workspace, s); }});
}}
// The reference signature has no workspace argument: a kv-splitting configuration runs unsplit here.
extern "C" float profile(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return -1.f;
  return aat::timed_mean_ms(nullptr, [&] {{ return launch(q, k, v, o, B, H, Seq_q, Seq_k, kReferenceScale, 0, nullptr, nullptr); }});
}}
"""

kernel_entry = r"""
extern "C" int kernel_entry_ex(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_q, int Seq_k,
                               float softmax_scale, int causal, void* workspace, size_t workspace_bytes, void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return AAT_ERR_SHAPE;
  if (split_applies(Seq_k, causal) && (workspace == nullptr || workspace_bytes < split_workspace_bytes(B, H, Seq_q)))
    return AAT_ERR_WORKSPACE;
  return (int)launch(q, k, v, o, B, H, Seq_q, Seq_k, softmax_scale, causal, workspace, static_cast<hipStream_t>(stream));
}}
extern "C" int kernel_entry(aat_half* q, aat_half* k, aat_half* v, aat_half* o, int B, int H, int Seq_k, int Seq_q) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return AAT_ERR_SHAPE;
  return (int)launch(q, k, v, o, B, H, Seq_q, Seq_k, kReferenceScale, 0, nullptr, nullptr);
}}
extern "C" int kernel_entry_lse(aat_half* q, aat_half* k, aat_half* v, aat_half* o, float* lse, int B, int H, int Seq_q,
                                int Seq_k, float softmax_scale, int causal, void* workspace, size_t workspace_bytes,
                                void* stream) {{
  if (!aat::shape_ok(B, H, Seq_q, Seq_k, Br, Bc)) return AAT_ERR_SHAPE;
  if (split_applies(Seq_k, causal) && (workspace == nullptr || workspace_bytes < split_workspace_bytes(B, H, Seq_q)))
    return AAT_ERR_WORKSPACE;
  return (int)launch(q, k, v, o, B, H, Seq_q, Seq_k, softmax_scale, causal, workspace, static_cast<hipStream_t>(stream), lse);
}}
"""

# One library carries both halves of the ABI, so tuning and running share a single compile.
profile_code = global_vars + profile_func + kernel_entry
kernel_code = profile_code
