// Flash-attention forward, register-fused variant, for gfx950 (MI355X).
//
// Computes O = softmax(scale * Q K^T) V with the online-softmax recurrence of the reference kernel
// (reference: csrc/kernels/attention/regfuse/regfuse.h:236-324 main loop, :407-453 epilogue): running
// UNSCALED row max m, l = l*alpha + rowsum(P), O = O*alpha + half(P) V, O /= l at the end; P is rounded
// to fp16 (RNE) before the second contraction and O is rounded to fp16 (RNE) on store.
//
// What is different from the reference, by design:
//  * transposed dataflow: S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_32x32x16_f16, so a lane owns one
//    query row; the C registers of S^T feed the second MFMA directly (that is the "register fuse");
//  * Q never touches LDS: it is loaded once, straight into MFMA B-operand registers;
//  * K and V tiles reach LDS by LDS-DMA (global_load_lds_dwordx4), XOR-swizzled, 1 or 2 buffers each;
//  * V^T operands come from ds_read_b64_tr_b16;
//  * the running max is lazy (softmax.h) and, in the pipelined schedule, the MFMAs of the NEXT score
//    tile are issued between the exponentials of the current one so matrix and vector pipes overlap
//    inside one wave;
//  * softmax scale and causal masking are runtime arguments (the reference hard-codes 0.125 at :50 and
//    has the causal bound commented out at :59-61).
#pragma once
#include <type_traits>

#include "../../utils/cdna4.h"
#include "../../utils/softmax.h"
#include "../../utils/tile_ops.h"

namespace aat {

template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV>
struct AttnFwdRegfuse {
  static constexpr int NW = Nthreads / kWave;   // waves per block
  static constexpr int WM = Br / NW;            // query rows per wave
  static constexpr int RT = WM / 32;            // 32-row groups per wave
  static constexpr int NT = Bc / 32;            // score tiles along kv
  static constexpr int KS = Kd / 16;            // MFMA k-steps of S^T = K Q^T
  static constexpr int DT = D / 32;             // output tiles along d
  static constexpr int NCK = Kd / 8, NCV = D / 8;
  static_assert(Nthreads % kWave == 0 && Br % NW == 0 && WM % 32 == 0, "each wave owns whole 32-row tiles");
  static_assert(Bc % 32 == 0 && Kd % 64 == 0 && D % 64 == 0, "tile shape");
  static_assert(NSK == 1 || NSK == 2, "K buffers");
  static_assert(NSV == 1 || NSV == 2, "V buffers");
  using KDma = TileDma<Bc, NCK, Nthreads, Swz::Rows16>;
  using VDma = TileDma<Bc, NCV, Nthreads, Swz::Rows4>;
  static constexpr int kKBytes = Bc * Kd * 2, kVBytes = Bc * D * 2;
  static constexpr int kOStride = D * 2 + 16;   // epilogue staging row stride (bytes)
  static constexpr int kMainBytes = NSK * kKBytes + NSV * kVBytes;
  static constexpr int kEpiBytes = Br * kOStride;
  static constexpr int kSmemBytes = kMainBytes > kEpiBytes ? kMainBytes : kEpiBytes;
};

// lse may be null.  When non-null it receives the natural-log-sum-exp of the scaled scores per row.
// PIPE selects the software-pipelined schedule (needs two K and two V buffers).
template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int WPE = 1, bool PIPE = false>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
flashattn_fwd_regfuse(const half_t* __restrict__ q, const half_t* __restrict__ k,
                      const half_t* __restrict__ v, half_t* __restrict__ o, float* __restrict__ lse,
                      int H, int seq_k, int seq_q, float softmax_scale, int causal) {
  using T = AttnFwdRegfuse<Kd, D, Br, Bc, Nthreads, NSK, NSV>;
  constexpr int RT = T::RT, NT = T::NT, KS = T::KS, DT = T::DT, NCK = T::NCK, NCV = T::NCV, WM = T::WM;
  static_assert(!PIPE || (NSK == 2 && NSV == 2), "the pipelined schedule reads K one tile ahead");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* const kbuf = smem;
  char* const vbuf = smem + NSK * T::kKBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;

  const int Tr = seq_q / Br;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = tile / Tr;
  int rb = tile % Tr;
  if (causal) rb = Tr - 1 - rb;                 // long rows first
  const int q0 = rb * Br;
  const int diag = seq_k - seq_q;               // kv index allowed for query i is <= i + diag
  int n_tiles = seq_k / Bc;
  int n_full = n_tiles;                         // tiles [0, n_full) are visible to every row of the block
  if (causal) {
    const int last = q0 + Br - 1 + diag;        // last visible kv index for this block
    const int lim = last < 0 ? 0 : last / Bc + 1;
    n_tiles = lim < n_tiles ? lim : n_tiles;
    const int full = (q0 + diag + 1) / Bc;
    n_full = full < 0 ? 0 : (full < n_tiles ? full : n_tiles);
  }

  const char* kg = reinterpret_cast<const char*>(k + (size_t)bh * seq_k * Kd);
  const char* vg = reinterpret_cast<const char*>(v + (size_t)bh * seq_k * D);

  typename T::KDma kdma;
  typename T::VDma vdma;
  kdma.init(tid, Kd * 2);
  vdma.init(tid, D * 2);
  const int wave_base = wave * 64;

  h8 qf[RT][KS];
  load_q_frags<RT, KS, Kd>(qf, q + ((size_t)bh * seq_q + q0 + wave * WM + n) * Kd + 8 * h);
  int koff[KS], voff[DT];
  k_frag_offsets<KS, NCK>(koff, n, h);
  v_frag_offsets<DT, NCV>(voff, lane);

  f16v oacc[RT][DT];
  float m_run[RT], l_run[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    m_run[rt] = -INFINITY;
    l_run[rt] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[rt][dt] = zero16();
  }
  const float c2 = softmax_scale * kLog2e;
  const int q_lim0 = q0 + wave * WM + n + diag;   // last kv index row n of row group 0 may see

  if constexpr (!PIPE) {
    // ============================ plain schedule =================================================
    if (n_tiles > 0) {
      kdma.issue(kg, kbuf, wave_base);
      if constexpr (NSV == 2) vdma.issue(vg, vbuf, wave_base);
    }
    auto kv_tile = [&](const int j, auto masked_tag) {
      constexpr bool MASKED = decltype(masked_tag)::value;
      char* const kcur = kbuf + (NSK == 2 ? (j & 1) * T::kKBytes : 0);
      char* const vcur = vbuf + (NSV == 2 ? (j & 1) * T::kVBytes : 0);
      const bool more = (j + 1 < n_tiles);

      // (A) K_j (and with two V buffers V_j) has landed; every wave is past iteration j-1.
      wait_vmcnt<0>();
      block_sync();
      if constexpr (NSV == 1) vdma.issue(vg + (size_t)j * T::kVBytes, vcur, wave_base);
      if (more) {
        if constexpr (NSK == 2) kdma.issue(kg + (size_t)(j + 1) * T::kKBytes, kbuf + ((j + 1) & 1) * T::kKBytes, wave_base);
        if constexpr (NSV == 2) vdma.issue(vg + (size_t)(j + 1) * T::kVBytes, vbuf + ((j + 1) & 1) * T::kVBytes, wave_base);
      }

      f16v sacc[RT][NT];
      qk_gemm<RT, NT, KS, NCK>(sacc, qf, kcur, koff);

      h8 pf[RT][NT][2];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int q_lim = q_lim0 + rt * 32;
        if constexpr (MASKED) causal_mask<NT>(sacc[rt], j * Bc, q_lim, h);
        const float mc = lazy_max_step<NT, DT>(sacc[rt], m_run[rt], l_run[rt], oacc[rt], c2);
        l_run[rt] += exp_tile<NT, MASKED>(sacc[rt], c2, mc, j * Bc, q_lim, h);   // per-lane partial sum
        pack_p<NT>(pf[rt], sacc[rt]);
      }

      // (B) with one buffer: V_j must have landed / K buffer must be free before K_{j+1} is fetched.
      if constexpr (NSV == 1 || NSK == 1) {
        if constexpr (NSV == 1) wait_vmcnt<0>();
        block_sync();
        if constexpr (NSK == 1) {
          if (more) kdma.issue(kg + (size_t)(j + 1) * T::kKBytes, kbuf, wave_base);
        }
      }
      pv_gemm<RT, NT, DT, NCV>(oacc, pf, vcur, voff);
    };
    for (int j = 0; j < n_full; ++j) kv_tile(j, std::false_type{});
    for (int j = n_full; j < n_tiles; ++j) kv_tile(j, std::true_type{});
  } else {
    // ============================ pipelined schedule =============================================
    // Iteration j holds S_j in registers (computed one iteration earlier) and does
    //   [ S_{j+1} = K_{j+1} Q^T  interleaved with  P_j = exp(S_j - m) ] ; O += V_j^T P_j.
    // Buffers: K_{j+1} is read while K_{j+2} is fetched into the other K buffer; V_j is read while
    // V_{j+1} is fetched.  One barrier per iteration.
    f16v scur[RT][NT];
    if (n_tiles > 0) {
      kdma.issue(kg, kbuf, wave_base);
      vdma.issue(vg, vbuf, wave_base);
      if (n_tiles > 1) kdma.issue(kg + T::kKBytes, kbuf + T::kKBytes, wave_base);
      wait_vmcnt<0>();
      block_sync();
      qk_gemm<RT, NT, KS, NCK>(scur, qf, kbuf, koff);
    }
    auto kv_tile = [&](const int j, auto masked_tag) {
      constexpr bool MASKED = decltype(masked_tag)::value;
      char* const knext = kbuf + ((j + 1) & 1) * T::kKBytes;
      char* const vcur = vbuf + (j & 1) * T::kVBytes;
      // K_{j+1} and V_j have landed; every wave finished S_j (frees K buffer j&1) and O += V_{j-1} P.
      wait_vmcnt<0>();
      block_sync();
      if (j + 2 < n_tiles) kdma.issue(kg + (size_t)(j + 2) * T::kKBytes, kbuf + (j & 1) * T::kKBytes, wave_base);
      if (j + 1 < n_tiles) vdma.issue(vg + (size_t)(j + 1) * T::kVBytes, vbuf + ((j + 1) & 1) * T::kVBytes, wave_base);

      float mc[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if constexpr (MASKED) causal_mask<NT>(scur[rt], j * Bc, q_lim0 + rt * 32, h);
        mc[rt] = lazy_max_step<NT, DT>(scur[rt], m_run[rt], l_run[rt], oacc[rt], c2);
      }

      f16v snext[RT][NT];
      h8 pf[RT][NT][2];
      if (j + 1 < n_tiles) {
        constexpr int kSteps = NT * KS;                              // MFMA groups of the next tile
        constexpr int kPerStep = (NT * 16 + kSteps - 1) / kSteps;    // exponentials per group and row group
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) snext[rt][nt] = zero16();
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
          qk_step<RT, NT, KS, NCK>(snext, qf, knext, koff, step / KS, step % KS);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            l_run[rt] += exp_range<NT, MASKED>(scur[rt], step * kPerStep, kPerStep, c2, mc[rt], j * Bc, q_lim0 + rt * 32, h);
        }
      } else {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          l_run[rt] += exp_tile<NT, MASKED>(scur[rt], c2, mc[rt], j * Bc, q_lim0 + rt * 32, h);
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) pack_p<NT>(pf[rt], scur[rt]);
      pv_gemm<RT, NT, DT, NCV>(oacc, pf, vcur, voff);
      if (j + 1 < n_tiles) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) scur[rt][nt] = snext[rt][nt];
      }
    };
    for (int j = 0; j < n_full; ++j) kv_tile(j, std::false_type{});
    for (int j = n_full; j < n_tiles; ++j) kv_tile(j, std::true_type{});
  }

  // ---- epilogue: normalise, round, transpose through LDS, coalesced store ----------------------
  wait_vmcnt<0>();
  block_sync();                                  // every wave is done with the K/V buffers
  float inv[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float l_tot = pair_sum(l_run[rt]);
    inv[rt] = l_tot > 0.f ? fast_rcp(l_tot) : 0.f;
    if (lse != nullptr && h == 0) {
      const size_t row = (size_t)bh * seq_q + q0 + wave * WM + rt * 32 + n;
      lse[row] = l_tot > 0.f ? m_run[rt] * softmax_scale + __logf(l_tot) : -INFINITY;
    }
  }
  store_o_tile<RT, DT, D, T::kOStride>(oacc, inv, smem + wave * WM * T::kOStride,
                                       o + ((size_t)bh * seq_q + q0 + wave * WM) * D, lane);
}

}  // namespace aat
