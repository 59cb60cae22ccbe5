// Flash-attention forward, LDS-fused variant, for gfx950 (MI355X).
//
// Same result as the register-fused kernel (attention/regfuse/regfuse.h); P travels through LDS so
// the second contraction can use its own wave grid (see utils/smemfuse.h).  Counterpart of reference
// csrc/kernels/attention/smemfuse/smemfuse.h:61-614.  Per kv tile:
//   1. every wave: S^T sub-tile = K_part Q_rows^T                       (registers)
//   2. partial row max -> LDS, barrier, combined max; lazy reference-point update
//   3. P = exp2(S*c - m*c) -> fp16 -> LDS; owner waves publish the rescale factor of their rows; barrier
//   4. every wave: O^T slice += V_slice^T P^T, rescaling first when some row moved its reference point
#pragma once
#include <type_traits>

#include "../../utils/cdna4.h"
#include "../../utils/smemfuse.h"
#include "../../utils/softmax.h"
#include "../../utils/tile_ops.h"

#ifndef AAT_PF
#define AAT_PF 2
#endif

namespace aat {

template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int W1N, int W2N>
struct AttnFwdSmemfuse {
  using G = SmemFuseGrid<Br, Bc, D, Nthreads, W1N, W2N>;
  static constexpr int KS = Kd / 16, NCK = Kd / 8, NCV = D / 8;
  static_assert(Kd % 64 == 0 && D % 64 == 0 && Bc % 32 == 0, "tile shape");
  static_assert((NSK == 1 || NSK == 2) && (NSV == 1 || NSV == 2), "buffers");
  using KDma = TileDma<Bc, NCK, Nthreads, Swz::Rows16>;
  using VDma = TileDma<Bc, NCV, Nthreads, Swz::Rows4>;
  static constexpr int kKBytes = Bc * Kd * 2, kVBytes = Bc * D * 2;
  static constexpr int kPOff = NSK * kKBytes + NSV * kVBytes;
  static constexpr int kStatOff = kPOff + G::kPBytes;
  static constexpr int kMainBytes = kStatOff + G::kStatBytes;
  static constexpr int kSmemBytes = kMainBytes > G::kEpiBytes ? kMainBytes : G::kEpiBytes;
};

template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int W1N, int W2N, int WPE = 1,
          bool CAUSAL = false>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
flashattn_fwd_smemfuse(const half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
                       half_t* __restrict__ o, float* __restrict__ lse, int H, int seq_k, int seq_q,
                       float softmax_scale) {
  using T = AttnFwdSmemfuse<Kd, D, Br, Bc, Nthreads, NSK, NSV, W1N, W2N>;
  using G = typename T::G;
  constexpr int RT1 = G::RT1, NT1 = G::NT1, RT2 = G::RT2, DT2 = G::DT2, KS = T::KS, NCK = T::NCK, NCV = T::NCV;
  constexpr int PF = AAT_PF;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* const kbuf = smem;
  char* const vbuf = smem + NSK * T::kKBytes;
  char* const pbuf = smem + T::kPOff;
  float* const part = reinterpret_cast<float*>(smem + T::kStatOff);      // [W1N][Br] partial row statistics
  float* const alpha_s = part + W1N * Br;                                  // [Br] rescale factor of the tile
  int* const flags = reinterpret_cast<int*>(alpha_s + Br);                 // [NW] "some row of this wave moved"

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int w1m = wave / W1N, w1n = wave % W1N;     // position in the first wave grid
  const int w2m = wave / W2N, w2n = wave % W2N;     // position in the second wave grid

  const int Tr = seq_q / Br;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  int bh = tile / Tr, rb = tile % Tr;
  if constexpr (CAUSAL) {
    const TileId t = causal_tile(blockIdx.x, gridDim.x, Tr, true);
    bh = t.bh;
    rb = t.blk;
  }
  const int q0 = rb * Br;
  const int diag = seq_k - seq_q;
  int n_tiles = seq_k / Bc;
  int n_full = n_tiles;
  if constexpr (CAUSAL) {
    const int last = q0 + Br - 1 + diag;
    const int lim = last < 0 ? 0 : last / Bc + 1;
    n_tiles = lim < n_tiles ? lim : n_tiles;
    const int full = (q0 + diag + 1) / Bc;
    n_full = full < 0 ? 0 : (full < n_tiles ? full : n_tiles);
    n_full &= ~1;
  }

  const char* kg = reinterpret_cast<const char*>(k + (size_t)bh * seq_k * Kd);
  const char* vg = reinterpret_cast<const char*>(v + (size_t)bh * seq_k * D);
  typename T::KDma kdma;
  typename T::VDma vdma;
  kdma.init(tid);
  vdma.init(tid);
  const int wave_base = wave * 64;

  // first contraction: this wave's rows and kv columns
  const int row1 = w1m * G::RM1;                   // first query row (within the block) of this wave
  h8 qf[RT1][KS];
  load_q_frags<RT1, KS, Kd>(qf, q + ((size_t)bh * seq_q + q0 + row1 + n) * Kd + 8 * h);
  uint32_t kaddr[KS];
  {
    int koff[KS];
    k_frag_offsets<KS, NCK>(koff, n, h);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds_addr(kbuf + w1n * G::CN1 * NCK * 16 + koff[ks]);
  }
  const uint32_t prow_w = lds_addr(pbuf + (row1 + n) * G::kPStride + (w1n * G::CN1) * 2 + 8 * h);
  // second contraction: this wave's rows and d columns
  const int row2 = w2m * G::RM2;
  uint32_t paddr[RT2], vaddr[DT2];
#pragma unroll
  for (int rt = 0; rt < RT2; ++rt) paddr[rt] = lds_addr(pbuf + (row2 + rt * 32 + n) * G::kPStride + 16 * h);
  v_frag_addrs_8<DT2, NCV>(vaddr, vbuf, lane, w2n * DT2);

  f16v oacc[RT2][DT2];
#pragma unroll
  for (int rt = 0; rt < RT2; ++rt)
#pragma unroll
    for (int dt = 0; dt < DT2; ++dt) oacc[rt][dt] = zero16();
  float m_run[RT1], l_run[RT1];
#pragma unroll
  for (int rt = 0; rt < RT1; ++rt) {
    m_run[rt] = -INFINITY;
    l_run[rt] = 0.f;
  }
  const float c2 = softmax_scale * kLog2e;
  const int q_lim0 = q0 + row1 + n + diag;

  if (n_tiles > 0) {
    kdma.issue(kg, kbuf, wave_base);
    if constexpr (NSV == 2) vdma.issue(vg, vbuf, wave_base);
  }
  auto kv_tile = [&](const int j, auto parity_tag, auto masked_tag) {
    constexpr int PAR = decltype(parity_tag)::value;
    constexpr bool MASKED = decltype(masked_tag)::value;
    const bool more = (j + 1 < n_tiles);
    // (A) K_j (and V_j with two V buffers) landed; all waves are past iteration j-1 (P, stats, buffers free).
    wait_vmcnt<0>();
    block_sync();
    if constexpr (NSV == 1) vdma.issue(vg + (size_t)j * T::kVBytes, vbuf, wave_base);
    if (more) {
      if constexpr (NSK == 2) kdma.issue(kg + (size_t)(j + 1) * T::kKBytes, kbuf + (PAR ^ 1) * T::kKBytes, wave_base);
      if constexpr (NSV == 2) vdma.issue(vg + (size_t)(j + 1) * T::kVBytes, vbuf + (PAR ^ 1) * T::kVBytes, wave_base);
    }

    f16v sacc[RT1][NT1];
    qk_gemm_steps<RT1, NT1, KS, NCK, PF>(sacc, qf, kaddr, NSK == 2 ? PAR * T::kKBytes : 0, [](int) {});
    const int kv0 = j * Bc + w1n * G::CN1;
    float m_tile[RT1];
#pragma unroll
    for (int rt = 0; rt < RT1; ++rt) {
      if constexpr (MASKED) causal_mask<NT1>(sacc[rt], kv0, q_lim0 + rt * 32, h);
      m_tile[rt] = pair_max(lane_max<NT1>(sacc[rt]));
    }
    if constexpr (W1N > 1) {
      // combine the partial row maxima of the W1N waves that share these rows
      if (h == 0) {
#pragma unroll
        for (int rt = 0; rt < RT1; ++rt) part[w1n * Br + row1 + rt * 32 + n] = m_tile[rt];
      }
      block_sync();
#pragma unroll
      for (int rt = 0; rt < RT1; ++rt) {
        float m = -INFINITY;
#pragma unroll
        for (int x = 0; x < W1N; ++x) m = fmaxf(m, part[x * Br + row1 + rt * 32 + n]);
        m_tile[rt] = m;
      }
    }
    bool moved = false;
#pragma unroll
    for (int rt = 0; rt < RT1; ++rt) {
      const bool grow = (m_tile[rt] - m_run[rt]) * c2 > kLazyLog2;
      float alpha = 1.f;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        const float m_new = fmaxf(m_run[rt], m_tile[rt]);
        const SoftmaxStep st = softmax_step(m_run[rt], m_new, c2);
        m_run[rt] = m_new;
        l_run[rt] *= st.alpha;
        alpha = st.alpha;
        moved = true;
      }
      if (w1n == 0 && h == 0) alpha_s[row1 + rt * 32 + n] = alpha;
      const float mc = (m_run[rt] == -INFINITY ? 0.f : m_run[rt]) * c2;
      exp_tile<NT1>(sacc[rt], c2, mc);
      if constexpr (MASKED) zero_masked<NT1>(sacc[rt], kv0, q_lim0 + rt * 32, h);
      float lsum = 0.f;
#pragma unroll
      for (int nt = 0; nt < NT1; ++nt)
#pragma unroll
        for (int vv = 0; vv < 16; ++vv) lsum += sacc[rt][nt][vv];
      l_run[rt] += lsum;
    }
    if (lane == 0) flags[wave] = moved ? 1 : 0;
    store_p<RT1, NT1, G::kPStride>(sacc, prow_w);

    // (B) P, rescale factors and flags are published; V_j has landed; K buffer is free.
    if constexpr (NSV == 1) wait_vmcnt<0>();
    block_sync();
    if constexpr (NSK == 1) {
      if (more) kdma.issue(kg + (size_t)(j + 1) * T::kKBytes, kbuf, wave_base);
    }
    int any = 0;
#pragma unroll
    for (int w = 0; w < G::NW; ++w) any |= flags[w];
    if (__builtin_amdgcn_readfirstlane(any) != 0) {
#pragma unroll
      for (int rt = 0; rt < RT2; ++rt) {
        const float a = alpha_s[row2 + rt * 32 + n];
#pragma unroll
        for (int dt = 0; dt < DT2; ++dt)
#pragma unroll
          for (int vv = 0; vv < 16; ++vv) oacc[rt][dt][vv] *= a;
      }
    }
    pv_gemm_from_lds<RT2, DT2, Bc / 16, NCV>(oacc, paddr, vaddr, NSV == 2 ? PAR * T::kVBytes : 0);
  };
  {
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    const int n_plain = CAUSAL ? n_full : n_tiles;
    for (int j = 0; j < n_plain; j += 2) {
      kv_tile(j, P0{}, std::false_type{});
      if (j + 1 < n_plain) kv_tile(j + 1, P1{}, std::false_type{});
    }
    if constexpr (CAUSAL) {
      for (int j = n_full; j < n_tiles; j += 2) {
        kv_tile(j, P0{}, std::true_type{});
        if (j + 1 < n_tiles) kv_tile(j + 1, P1{}, std::true_type{});
      }
    }
  }

  // ---- epilogue: combine the row sums, normalise, store ---------------------------------------------
  wait_vmcnt<0>();
  block_sync();
#pragma unroll
  for (int rt = 0; rt < RT1; ++rt) {
    const float l_w = pair_sum(l_run[rt]);
    if (h == 0) part[w1n * Br + row1 + rt * 32 + n] = l_w;
    if (w1n == 0 && h == 0) alpha_s[row1 + rt * 32 + n] = m_run[rt];
  }
  block_sync();
  float inv[RT2];
#pragma unroll
  for (int rt = 0; rt < RT2; ++rt) {
    float l_tot = 0.f;
#pragma unroll
    for (int x = 0; x < W1N; ++x) l_tot += part[x * Br + row2 + rt * 32 + n];
    inv[rt] = l_tot > 0.f ? fast_rcp(l_tot) : 0.f;
    if (lse != nullptr && h == 0 && w2n == 0) {
      const float m_fin = alpha_s[row2 + rt * 32 + n];
      lse[(size_t)bh * seq_q + q0 + row2 + rt * 32 + n] = l_tot > 0.f ? m_fin * softmax_scale + __logf(l_tot) : -INFINITY;
    }
  }
  block_sync();                                   // statistics read; the staging area may overwrite them
  store_o_slice<RT2, DT2, D, G::kOStride>(oacc, inv, smem + wave * G::RM2 * G::kOStride,
                                          o + ((size_t)bh * seq_q + q0 + row2) * D + w2n * G::DN2, lane);
}

}  // namespace aat
