// RetNet parallel retention forward, LDS-fused variant, for gfx950 (MI355X).
//
// Same result as the register-fused kernel (retnet/regfuse/regfuse.h); P travels through LDS so the
// second contraction can use its own wave grid (utils/smemfuse.h) -- the variant of choice for wide
// value heads (d_v = 512 keeps 128 accumulator registers per lane with Br = 64 and four waves).
// Counterpart of reference csrc/kernels/retnet/smemfuse/smemfuse.h:62-635.  Per kv tile:
//   1. every wave: S^T sub-tile = (K_part Q_rows^T) * mask_part        (registers)
//   2. partial abs-sums -> LDS, barrier, R += total; lazy move of the scale r_ref (utils/retention.h)
//   3. P = S / r_ref -> fp16 -> LDS; owner waves publish the rescale factor of their rows; barrier
//   4. every wave: O^T slice += V_slice^T P^T, rescaling first when some row moved its scale
#pragma once
#include <type_traits>

#include "../../utils/cdna4.h"
#include "../../utils/mask_extents.h"
#include "../../utils/retention.h"
#include "../../utils/smemfuse.h"
#include "../../utils/tile_ops.h"

#ifndef AAT_PF
#define AAT_PF 2
#endif

namespace aat {

template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int NSM, int W1N, int W2N>
struct RetFwdSmemfuse {
  using G = SmemFuseGrid<Br, Bc, D, Nthreads, W1N, W2N>;
  static constexpr int KS = Kd / 16, NCK = Kd / 8, NCV = D / 8, NCM = Bc / 8;
  static_assert(Kd % 64 == 0 && D % 64 == 0 && Bc % 32 == 0, "tile shape");
  static_assert((NSK == 1 || NSK == 2) && (NSV == 1 || NSV == 2) && (NSM == 1 || NSM == 2) && NSM >= NSK, "buffers");
  using KDma = TileDma<Bc, NCK, Nthreads, Swz::Rows16>;
  using VDma = TileDma<Bc, NCV, Nthreads, Swz::Rows4>;
  using MDma = TileDma<Br, NCM, Nthreads, Swz::Rows16>;
  static constexpr int kKBytes = Bc * Kd * 2, kVBytes = Bc * D * 2, kMBytes = Br * Bc * 2;
  static constexpr int kMOff = NSK * kKBytes + NSV * kVBytes;
  static constexpr int kPOff = kMOff + NSM * kMBytes;
  static constexpr int kStatOff = kPOff + G::kPBytes;
  static constexpr int kMainBytes = kStatOff + G::kStatBytes;
  static constexpr int kSmemBytes = kMainBytes > G::kEpiBytes ? kMainBytes : G::kEpiBytes;
};

// DECAY: the mask is gamma_h^(q + diag - kv) below the diagonal and zero above it, built in registers
// from lg2gamma[h] = log2(gamma_h); `mask` is not read and tiles above the diagonal are skipped.
template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int NSM, int W1N, int W2N, int WPE = 1,
          bool DECAY = false>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
ret_fwd_smemfuse(const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
                 const half_t* __restrict__ mask, half_t* __restrict__ o, float* __restrict__ r, int H,
                 int seq_k, int seq_q, int causal, const float* __restrict__ lg2gamma = nullptr,
                 const int* __restrict__ extents = nullptr) {
  if constexpr (DECAY) causal = 1;
  using T = RetFwdSmemfuse<Kd, D, Br, Bc, Nthreads, NSK, NSV, NSM, W1N, W2N>;
  using G = typename T::G;
  constexpr int RT1 = G::RT1, NT1 = G::NT1, RT2 = G::RT2, DT2 = G::DT2, KS = T::KS, NCK = T::NCK, NCV = T::NCV, NCM = T::NCM;
  constexpr int PF = AAT_PF;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* const kbuf = smem;
  char* const vbuf = smem + NSK * T::kKBytes;
  char* const mbuf = smem + T::kMOff;
  char* const pbuf = smem + T::kPOff;
  float* const part = reinterpret_cast<float*>(smem + T::kStatOff);      // [W1N][Br]
  float* const alpha_s = part + W1N * Br;                                  // [Br]
  int* const flags = reinterpret_cast<int*>(alpha_s + Br);                 // [NW]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int w1m = wave / W1N, w1n = wave % W1N;
  const int w2m = wave / W2N, w2n = wave % W2N;

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
  DecayMask<NT1, true> decay;
  if constexpr (DECAY) decay.init(lg2gamma[bh % H], h);
  typename T::KDma kdma;
  typename T::VDma vdma;
  typename T::MDma mdma;
  kdma.init(tid);
  vdma.init(tid);
  mdma.init(tid, seq_k * 2);
  const int wave_base = wave * 64;

  const int row1 = w1m * G::RM1;
  h8 qf[RT1][KS];
  load_q_frags<RT1, KS, Kd>(qf, q + ((size_t)bh * seq_q + q0 + row1 + n) * Kd + 8 * h);
  uint32_t kaddr[KS], maddr[RT1][NT1 * 4];
  {
    int koff[KS];
    k_frag_offsets<KS, NCK>(koff, n, h);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds_addr(kbuf + w1n * G::CN1 * NCK * 16 + koff[ks]);
#pragma unroll
    for (int rt = 0; rt < RT1; ++rt)
#pragma unroll
      for (int i = 0; i < NT1 * 4; ++i)
        maddr[rt][i] = lds_addr(mbuf + lds_chunk_off<NCM, Swz::Rows16>(row1 + rt * 32 + n, w1n * (G::CN1 / 8) + i) + 8 * h);
  }
  const uint32_t prow_w = lds_addr(pbuf + (row1 + n) * G::kPStride + (w1n * G::CN1) * 2 + 8 * h);
  const int row2 = w2m * G::RM2;
  uint32_t paddr[RT2], vaddr[DT2];
#pragma unroll
  for (int rt = 0; rt < RT2; ++rt) paddr[rt] = lds_addr(pbuf + (row2 + rt * 32 + n) * G::kPStride + 16 * h);
  v_frag_addrs_8<DT2, NCV>(vaddr, vbuf, lane, w2n * DT2);

  f16v oacc[RT2][DT2];
#pragma unroll
  for (int rt = 0; rt < RT2; ++rt)
#pragma unroll
    for (int dt = 0; dt < DT2; ++dt) {
      oacc[rt][dt] = zero16();
      // one wave per SIMD: zero into accumulation registers, or the literal zeros that also reach the epilogue on
      // the path of a block without kv tiles are kept in vector registers across the main loop
      if constexpr (WPE == 1) asm volatile("" : "+a"(oacc[rt][dt]));
    }
  RetentionRow row[RT1];
#pragma unroll
  for (int rt = 0; rt < RT1; ++rt) {
    row[rt].big_r = 0.f;
    row[rt].r_ref = 1.f;
  }

  auto issue_km = [&](int j, int par) {
    kdma.issue(kg + (size_t)j * T::kKBytes, kbuf + (NSK == 2 ? par * T::kKBytes : 0), wave_base);
    if constexpr (!DECAY) mdma.issue(mg + (size_t)j * Bc * 2, mbuf + (NSM == 2 ? par * T::kMBytes : 0), wave_base);
  };
  if (n_tiles > 0) {
    issue_km(0, 0);
    if constexpr (NSV == 2) vdma.issue(vg, vbuf, wave_base);
  }
  auto kv_tile = [&](const int j, auto parity_tag) {
    constexpr int PAR = decltype(parity_tag)::value;
    const bool more = (j + 1 < n_tiles);
    wait_vmcnt<0>();
    block_sync();
    if constexpr (NSV == 1) vdma.issue(vg + (size_t)j * T::kVBytes, vbuf, wave_base);
    if (more) {
      if constexpr (NSK == 2) issue_km(j + 1, PAR ^ 1);
      if constexpr (NSV == 2) vdma.issue(vg + (size_t)(j + 1) * T::kVBytes, vbuf + (PAR ^ 1) * T::kVBytes, wave_base);
    }

    f16v sacc[RT1][NT1];
    qk_gemm_steps<RT1, NT1, KS, NCK, PF>(sacc, qf, kaddr, NSK == 2 ? PAR * T::kKBytes : 0, [](int) {});
    float tile_abs[RT1];
#pragma unroll
    for (int rt = 0; rt < RT1; ++rt) {
      if constexpr (DECAY) {
        const int own0 = q0 + row1 + rt * 32 + diag;                   // q + diag of the group's first row
        const int kv_org = j * Bc + w1n * G::CN1;                       // first kv column of this wave's score tiles
        const auto one = [](int, int) { return 1.0f; };
        if (kv_org + G::CN1 - 1 > own0) decay.template apply<true>(sacc[rt], own0 + n - kv_org, one);
        else decay.template apply<false>(sacc[rt], own0 + n - kv_org, one);
      } else {
        apply_mask<NT1>(sacc[rt], maddr[rt], NSM == 2 ? PAR * T::kMBytes : 0);
      }
      float a = 0.f;
#pragma unroll
      for (int nt = 0; nt < NT1; ++nt)
#pragma unroll
        for (int vv = 0; vv < 16; ++vv) a += __builtin_fabsf(sacc[rt][nt][vv]);
      tile_abs[rt] = pair_sum(a);
    }
    if constexpr (W1N > 1) {
      if (h == 0) {
#pragma unroll
        for (int rt = 0; rt < RT1; ++rt) part[w1n * Br + row1 + rt * 32 + n] = tile_abs[rt];
      }
      block_sync();
#pragma unroll
      for (int rt = 0; rt < RT1; ++rt) {
        float a = 0.f;
#pragma unroll
        for (int x = 0; x < W1N; ++x) a += part[x * Br + row1 + rt * 32 + n];
        tile_abs[rt] = a;
      }
    }
    bool moved = false;
#pragma unroll
    for (int rt = 0; rt < RT1; ++rt) {
      row[rt].big_r += tile_abs[rt];
      const bool grow = row[rt].big_r > kLazyRatio * row[rt].r_ref;
      float alpha = 1.f;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        const float r_new = fmaxf(row[rt].big_r, 1.0f);
        alpha = row[rt].r_ref * fast_rcp(r_new);
        row[rt].r_ref = r_new;
        moved = true;
      }
      if (w1n == 0 && h == 0) alpha_s[row1 + rt * 32 + n] = alpha;
      const float inv = fast_rcp(row[rt].r_ref);
#pragma unroll
      for (int nt = 0; nt < NT1; ++nt)
#pragma unroll
        for (int vv = 0; vv < 16; ++vv) sacc[rt][nt][vv] *= inv;
    }
    if (lane == 0) flags[wave] = moved ? 1 : 0;
    store_p<RT1, NT1, G::kPStride>(sacc, prow_w);

    if constexpr (NSV == 1) wait_vmcnt<0>();
    block_sync();
    if constexpr (NSK == 1) {
      if (more) issue_km(j + 1, 0);
    }
    int any = 0;
#pragma unroll
    for (int w = 0; w < G::NW; ++w) any |= flags[w];
    if (__builtin_amdgcn_readfirstlane(any) != 0) {
#pragma unroll
      for (int rt = 0; rt < RT2; ++rt) {
        rescale_acc<DT2, WPE == 1>(oacc[rt], alpha_s[row2 + rt * 32 + n]);
      }
    }
    pv_gemm_from_lds<RT2, DT2, Bc / 16, NCV>(oacc, paddr, vaddr, NSV == 2 ? PAR * T::kVBytes : 0);
  };
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  for (int j = 0; j < n_tiles; j += 2) {
    kv_tile(j, P0{});
    if (j + 1 < n_tiles) kv_tile(j + 1, P1{});
  }

  // ---- epilogue: exact normaliser, r output, store ------------------------------------------------------
  wait_vmcnt<0>();
  block_sync();
#pragma unroll
  for (int rt = 0; rt < RT1; ++rt) {
    const float r_fin = fmaxf(row[rt].big_r, 1.0f);
    if (w1n == 0 && h == 0) {
      alpha_s[row1 + rt * 32 + n] = row[rt].r_ref * fast_rcp(r_fin);
      r[(size_t)bh * seq_q + q0 + row1 + rt * 32 + n] = r_fin;
    }
  }
  block_sync();
  float scale[RT2];
#pragma unroll
  for (int rt = 0; rt < RT2; ++rt) scale[rt] = alpha_s[row2 + rt * 32 + n];
  block_sync();                                   // statistics read; the staging area may overwrite them
  store_o_slice<RT2, DT2, D, G::kOStride>(oacc, scale, smem + wave * G::RM2 * G::kOStride,
                                          o + ((size_t)bh * seq_q + q0 + row2) * D + w2n * G::DN2, lane);
}

}  // namespace aat
