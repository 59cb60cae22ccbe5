// RetNet parallel retention forward, register-fused variant, for gfx950 (MI355X).
//
//   S = (Q K^T) * mask,   r = max(sum_j |S|, 1),   O = (S / r) V        mask: [H, S_q, S_kv] fp16
//
// writes O (fp16) and r (fp32), as the reference kernel does (reference:
// csrc/kernels/retnet/regfuse/regfuse.h:267-340 main loop, :444-457 r store).  Same transposed MFMA dataflow
// and LDS-DMA staging as the attention kernel (attention/regfuse/regfuse.h); the mask tile travels
// through LDS as a third DMA stream, and the normalisation is lazy (utils/retention.h).
// `causal` promises a mask that is zero above the diagonal and only shortens the kv walk.
#pragma once
#include <type_traits>

#include "../../utils/acc_file.h"
#include "../../utils/cdna4.h"
#include "../../utils/mask_extents.h"
#include "../../utils/retention.h"
#include "../../utils/tile_ops.h"

#ifndef AAT_PF
#define AAT_PF 2
#endif

namespace aat {

template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int NSM>
struct RetFwdRegfuse {
  static constexpr int NW = Nthreads / kWave;
  static constexpr int WM = Br / NW;
  static constexpr int RT = WM / 32;
  static constexpr int NT = Bc / 32;
  static constexpr int KS = Kd / 16;
  static constexpr int DT = D / 32;
  static constexpr int NCK = Kd / 8, NCV = D / 8, NCM = Bc / 8;
  static_assert(Nthreads % kWave == 0 && Br % NW == 0 && WM % 32 == 0, "each wave owns whole 32-row tiles");
  static_assert(Bc % 32 == 0 && Kd % 64 == 0 && D % 64 == 0, "tile shape");
  static_assert((NSK == 1 || NSK == 2) && (NSV == 1 || NSV == 2) && (NSM == 1 || NSM == 2), "buffers");
  static_assert(NSM >= NSK, "the mask tile is consumed right after the K tile and is fetched with it");
  using KDma = TileDma<Bc, NCK, Nthreads, Swz::Rows16>;
  using VDma = TileDma<Bc, NCV, Nthreads, Swz::Rows4>;
  using MDma = TileDma<Br, NCM, Nthreads, Swz::Rows16>;
  static constexpr int kKBytes = Bc * Kd * 2, kVBytes = Bc * D * 2, kMBytes = Br * Bc * 2;
  static constexpr int kOStride = D * 2 + 16;
  static constexpr int kMainBytes = NSK * kKBytes + NSV * kVBytes + NSM * kMBytes;
  static constexpr int kEpiBytes = Br * kOStride;
  static constexpr int kSmemBytes = kMainBytes > kEpiBytes ? kMainBytes : kEpiBytes;
};

// DECAY: the mask is gamma_h^(q + diag - kv) below the diagonal and zero above it, built in registers
// from lg2gamma[h] = log2(gamma_h); `mask` is not read and tiles above the diagonal are skipped.
template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int NSM, int WPE = 1, bool DECAY = false>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
ret_fwd_regfuse(const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
                const half_t* __restrict__ mask, half_t* __restrict__ o, float* __restrict__ r, int H,
                int seq_k, int seq_q, int causal, const float* __restrict__ lg2gamma = nullptr,
                const int* __restrict__ extents = nullptr) {
  // One wave per SIMD: the output tile lives in the accumulation registers by number (utils/acc_file.h), the score
  // tile in vector registers through hand-written matrix instructions, and the compiler allocates the rest.
  constexpr bool kNumbered = WPE == 1;
  if constexpr (kNumbered) acc_claim_all();
  if constexpr (DECAY) causal = 1;
  using T = RetFwdRegfuse<Kd, D, Br, Bc, Nthreads, NSK, NSV, NSM>;
  constexpr int RT = T::RT, NT = T::NT, KS = T::KS, DT = T::DT, NCK = T::NCK, NCV = T::NCV, NCM = T::NCM, WM = T::WM;
  constexpr int PF = AAT_PF;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* const kbuf = smem;
  char* const vbuf = smem + NSK * T::kKBytes;
  char* const mbuf = vbuf + NSV * T::kVBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;

  const int Tr = seq_q / Br;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  int bh = tile / Tr, rb = tile % Tr;
  if (causal || extents != nullptr) {             // a scanned mask is taken to be of the causal kind: later rows see more
    const TileId t = causal_tile(blockIdx.x, gridDim.x, Tr, true);
    bh = t.bh;
    rb = t.blk;
  }
  const int q0 = rb * Br;
  int n_tiles = seq_k / Bc;
  if (extents != nullptr) {                       // walk up to the last kv tile in which the mask has a non-zero entry
    int lo, hi, j_begin;
    mask_row_range(mask_extents_at(extents, H, seq_q, seq_k), bh % H, seq_q, q0, Br, lo, hi);
    mask_tile_range(lo, hi, Bc, n_tiles, j_begin, n_tiles);
  } else if (causal) {
    const int last = q0 + Br - 1 + (seq_k - seq_q);
    const int lim = last < 0 ? 0 : last / Bc + 1;
    n_tiles = lim < n_tiles ? lim : n_tiles;
  }

  const char* kg = reinterpret_cast<const char*>(k + (size_t)bh * seq_k * Kd);
  const char* vg = reinterpret_cast<const char*>(v + (size_t)bh * seq_k * D);
  const char* mg = DECAY ? nullptr : reinterpret_cast<const char*>(mask + ((size_t)(bh % H) * seq_q + q0) * seq_k);
  const int diag = seq_k - seq_q;
  DecayMask<NT, true> decay;
  if constexpr (DECAY) decay.init(lg2gamma[bh % H], h);

  typename T::KDma kdma;
  typename T::VDma vdma;
  typename T::MDma mdma;
  kdma.init(tid);
  vdma.init(tid);
  mdma.init(tid, seq_k * 2);
  const int wave_base = wave * 64;

  h8 qf[RT][KS];
  load_q_frags<RT, KS, Kd>(qf, q + ((size_t)bh * seq_q + q0 + wave * WM + n) * Kd + 8 * h);
  // one mask address per 32-row group where the tile's rows are a power of two of chunks (see apply_mask_folded)
  constexpr bool kFoldMask = (NCM & (NCM - 1)) == 0 && NCM <= 16;
  uint32_t kaddr[KS], vaddr[DT], maddr[RT][kFoldMask ? 1 : NT * 4];
  {
    int koff[KS], voff[DT];
    k_frag_offsets<KS, NCK>(koff, n, h);
    v_frag_offsets<DT, NCV>(voff, lane);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds_addr(kbuf + koff[ks]);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vaddr[dt] = lds_addr(vbuf + voff[dt]);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < (kFoldMask ? 1 : NT * 4); ++i)
        maddr[rt][i] = lds_addr(mbuf + lds_chunk_off<NCM, Swz::Rows16>(wave * WM + rt * 32 + n, i) + 8 * h);
  }

  RetentionRow row[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    row[rt].big_r = 0.f;
    row[rt].r_ref = 1.f;
  }
  auto issue_km = [&](int j, int par) {          // K tile j and mask tile j travel together
    kdma.issue(kg + (size_t)j * T::kKBytes, kbuf + (NSK == 2 ? par * T::kKBytes : 0), wave_base);
    if constexpr (!DECAY) mdma.issue(mg + (size_t)j * Bc * 2, mbuf + (NSM == 2 ? par * T::kMBytes : 0), wave_base);
  };
  if (n_tiles > 0) {
    issue_km(0, 0);
    if constexpr (NSV == 2) vdma.issue(vg, vbuf, wave_base);
  }

  if constexpr (kNumbered) {
    static_assert(RT * DT * 16 <= 256, "a wave's output tile fills at most the accumulation file");
    acc_zero<0, RT * DT * 16>();
    // The copies of a tile are issued one instruction at a time between the matrix steps: a burst of them fills the
    // memory pipeline's queue, and the wave -- the only one on its SIMD -- stands still with an idle matrix pipe until
    // the queue has taken the last of them.
    constexpr int KI = T::KDma::kIters, VI = T::VDma::kIters, MI = DECAY ? 0 : T::MDma::kIters;
    auto issue_km_one = [&](int j, int par, int i) {          // instruction i of the K copy followed by the mask copy
      if (i < KI) kdma.issue_one(i, kg + (size_t)j * T::kKBytes, kbuf + (NSK == 2 ? par * T::kKBytes : 0), wave_base);
      else if constexpr (!DECAY) mdma.issue_one(i - KI, mg + (size_t)j * Bc * 2, mbuf + (NSM == 2 ? par * T::kMBytes : 0), wave_base);
    };
    // One loop body for both buffer parities: the parity is a run-time value that moves the operand addresses and the
    // copy destinations.
    int par = 0;
    for (int j = 0; j < n_tiles; ++j) {
      const bool more = (j + 1 < n_tiles);
      // (A) K_j, mask_j (and with two V buffers V_j) have landed; every wave is past iteration j-1.
      wait_vmcnt<0>();
      block_sync();
      f16v sacc[RT][NT];
      // between the steps of the first contraction: V_j into a single V buffer, K_j+1 and mask_j+1 into second buffers
      qk_gemm_steps<RT, NT, KS, NCK, PF, true>(sacc, qf, kaddr, 0, [&](int step) {
        constexpr int kSteps = NT * KS, kOwnV = NSV == 1 ? VI : 0, kCopies = kOwnV + (NSK == 2 ? KI + MI : 0);
        constexpr int kPer = (kCopies + kSteps - 1) / kSteps;
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
          const int i = step * kPer + u;
          if (i < kOwnV) vdma.issue_one(i, vg + (size_t)j * T::kVBytes, vbuf, wave_base);
          else if (i < kCopies && more) issue_km_one(j + 1, par ^ 1, i - kOwnV);
        }
      });
      static_for<RT>([&](auto rt_tag) {
        constexpr int rt = decltype(rt_tag)::value;
        if constexpr (DECAY) {
          const int own0 = q0 + wave * WM + rt * 32 + diag;              // q + diag of the group's first row
          const auto one = [](int, int) { return 1.0f; };
          if ((j + 1) * Bc - 1 > own0) decay.template apply<true>(sacc[rt], own0 + n - j * Bc, one);
          else decay.template apply<false>(sacc[rt], own0 + n - j * Bc, one);
        } else {
          if constexpr (kFoldMask) apply_mask_folded_blind<NT>(sacc[rt], maddr[rt][0]);
          else apply_mask<NT>(sacc[rt], maddr[rt], 0);
        }
        // the matrix instructions that last wrote the output tile are a whole score contraction back
        retention_step_with<NT>(sacc[rt], row[rt], [&](float alpha) { acc_scale<16 * rt * DT, 16 * DT>(alpha); });
      });
      // (B) with one buffer: V_j must have landed / K and mask buffers must be free before the next fetch.
      if constexpr (NSV == 1 || NSK == 1) {
        if constexpr (NSV == 1) wait_vmcnt<0>();
        block_sync();
      }
      h8 pf[RT][NT][2];
      // between the steps of the second contraction: K_j+1 and mask_j+1 into single buffers (free since (B)), V_j+1 into
      // the second V buffer (free since (A))
      pv_gemm_steps_numbered<RT, NT, DT, NCV, PF, 0>(pf, vaddr, 0, [&](int g) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) pack_group<NT>(pf[rt], sacc[rt], g);
      }, [&](int step) {
        constexpr int kSteps = 2 * NT * DT, kKm = NSK == 1 ? KI + MI : 0, kCopies = kKm + (NSV == 2 ? VI : 0);
        constexpr int kEvery = (kCopies > 0 && kSteps >= 2 * kCopies) ? kSteps / kCopies : 1;     // few copies: spread out
        constexpr int kPer = (kCopies * kEvery + kSteps - 1) / kSteps;
        if (step % kEvery != 0 || !more) return;
#pragma unroll
        for (int u = 0; u < kPer; ++u) {
          const int i = (step / kEvery) * kPer + u;
          if (i < kKm) issue_km_one(j + 1, 0, i);
          else if (i < kCopies) vdma.issue_one(i - kKm, vg + (size_t)(j + 1) * T::kVBytes, vbuf + (par ^ 1) * T::kVBytes, wave_base);
        }
      });
      // the next tile reads the other buffers
      if constexpr (NSK == 2) {
        const int dk = par ? -T::kKBytes : T::kKBytes;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) kaddr[ks] += dk;
      }
      if constexpr (NSV == 2) {
        const int dv = par ? -T::kVBytes : T::kVBytes;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vaddr[dt] += dv;
      }
      if constexpr (NSM == 2 && !DECAY) {
        const int dm = par ? -T::kMBytes : T::kMBytes;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int i = 0; i < (kFoldMask ? 1 : NT * 4); ++i) maddr[rt][i] += dm;
      }
      par ^= 1;
    }
    acc_settle();
    wait_vmcnt<0>();
    block_sync();
    float scale[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const float r_fin = fmaxf(row[rt].big_r, 1.0f);
      scale[rt] = row[rt].r_ref * fast_rcp(r_fin);
      if (h == 0) r[(size_t)bh * seq_q + q0 + wave * WM + rt * 32 + n] = r_fin;
    }
    store_o_tile_numbered<RT, DT, D, T::kOStride, 0>(scale, smem + wave * WM * T::kOStride,
                                                     o + ((size_t)bh * seq_q + q0 + wave * WM) * D, lane);
    return;
  }

  f16v oacc[RT][DT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) oacc[rt][dt] = zero16();
  auto kv_tile = [&](const int j, auto parity_tag) {
    constexpr int PAR = decltype(parity_tag)::value;
    char* const vcur = vbuf + (NSV == 2 ? PAR * T::kVBytes : 0);
    const bool more = (j + 1 < n_tiles);

    // (A) K_j, mask_j (and with two V buffers V_j) have landed; every wave is past iteration j-1.
    wait_vmcnt<0>();
    block_sync();
    if constexpr (NSV == 1) vdma.issue(vg + (size_t)j * T::kVBytes, vcur, wave_base);
    if (more) {
      if constexpr (NSK == 2) issue_km(j + 1, PAR ^ 1);
      if constexpr (NSV == 2) vdma.issue(vg + (size_t)(j + 1) * T::kVBytes, vbuf + (PAR ^ 1) * T::kVBytes, wave_base);
    }

    f16v sacc[RT][NT];
    qk_gemm_steps<RT, NT, KS, NCK, PF>(sacc, qf, kaddr, NSK == 2 ? PAR * T::kKBytes : 0, [](int) {});
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if constexpr (DECAY) {
        const int own0 = q0 + wave * WM + rt * 32 + diag;              // q + diag of the group's first row
        const auto one = [](int, int) { return 1.0f; };
        if ((j + 1) * Bc - 1 > own0) decay.template apply<true>(sacc[rt], own0 + n - j * Bc, one);
        else decay.template apply<false>(sacc[rt], own0 + n - j * Bc, one);
      } else {
        if constexpr (kFoldMask) apply_mask_folded<NT>(sacc[rt], maddr[rt][0], NSM == 2 ? PAR * T::kMBytes : 0);
        else apply_mask<NT>(sacc[rt], maddr[rt], NSM == 2 ? PAR * T::kMBytes : 0);
      }
      retention_step<NT, DT>(sacc[rt], row[rt], oacc[rt]);
    }

    // (B) with one buffer: V_j must have landed / K and mask buffers must be free before the next fetch.
    if constexpr (NSV == 1 || NSK == 1) {
      if constexpr (NSV == 1) wait_vmcnt<0>();
      block_sync();
      if constexpr (NSK == 1) {
        if (more) issue_km(j + 1, 0);
      }
    }
    h8 pf[RT][NT][2];
    pv_gemm_steps<RT, NT, DT, NCV, PF>(oacc, pf, vaddr, NSV == 2 ? PAR * T::kVBytes : 0, [&](int g) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) pack_group<NT>(pf[rt], sacc[rt], g);
    });
  };
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  for (int j = 0; j < n_tiles; j += 2) {
    kv_tile(j, P0{});
    if (j + 1 < n_tiles) kv_tile(j + 1, P1{});
  }

  // ---- epilogue -------------------------------------------------------------------------------------
  wait_vmcnt<0>();
  block_sync();
  float scale[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float r_fin = fmaxf(row[rt].big_r, 1.0f);
    scale[rt] = row[rt].r_ref * fast_rcp(r_fin);
    if (h == 0) r[(size_t)bh * seq_q + q0 + wave * WM + rt * 32 + n] = r_fin;
  }
  store_o_tile<RT, DT, D, T::kOStride>(oacc, scale, smem + wave * WM * T::kOStride,
                                       o + ((size_t)bh * seq_q + q0 + wave * WM) * D, lane);
}

}  // namespace aat
