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
//  * softmax scale and causal masking are runtime arguments (the reference hard-codes 0.125 at :50 and
//    has the causal bound commented out at :59-61).
#pragma once
#include "../../utils/cdna4.h"
#include "../../utils/softmax.h"
#include <type_traits>

namespace aat {

template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV>
struct AttnFwdRegfuse {
  static constexpr int NW = Nthreads / kWave;   // waves per block
  static constexpr int WM = Br / NW;            // query rows per wave
  static constexpr int RT = WM / 32;            // 32-row sub-tiles per wave
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

// lse may be null.  When non-null it receives natural-log-sum-exp of the scaled scores per row, fp32.
// kv_begin/kv_end restrict the kv range (in tiles of Bc) a block walks: used by the split-KV launcher,
// which then also passes `part` (0-based split index) so O and lse go to the partial buffers.
template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int WPE = 1>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
flashattn_fwd_regfuse(const half_t* __restrict__ q, const half_t* __restrict__ k,
                      const half_t* __restrict__ v, half_t* __restrict__ o, float* __restrict__ lse,
                      int H, int seq_k, int seq_q, float softmax_scale, int causal) {
  using T = AttnFwdRegfuse<Kd, D, Br, Bc, Nthreads, NSK, NSV>;
  constexpr int RT = T::RT, NT = T::NT, KS = T::KS, DT = T::DT, NCK = T::NCK, NCV = T::NCV, WM = T::WM;
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
  if (causal) {
    const int last = q0 + Br - 1 + diag;        // last visible kv index for this block
    const int lim = last < 0 ? 0 : last / Bc + 1;
    n_tiles = lim < n_tiles ? lim : n_tiles;
  }

  const char* kg = reinterpret_cast<const char*>(k + (size_t)bh * seq_k * Kd);
  const char* vg = reinterpret_cast<const char*>(v + (size_t)bh * seq_k * D);

  typename T::KDma kdma;
  typename T::VDma vdma;
  kdma.init(tid, Kd * 2);
  vdma.init(tid, D * 2);
  const int wave_base = wave * 64;

  // ---- Q: straight from HBM into B-operand registers -------------------------------------------
  h8 qf[RT][KS];
  {
    const half_t* qrow = q + ((size_t)bh * seq_q + q0 + wave * WM + n) * Kd + 8 * h;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[rt][ks] = *reinterpret_cast<const h8*>(qrow + (size_t)rt * 32 * Kd + 16 * ks);
  }

  // ---- per-lane LDS read offsets --------------------------------------------------------------
  // K fragment (A operand): row n of score tile nt, chunk 2*ks + h.
  int koff[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff[ks] = lds_chunk_off<NCK, Swz::Rows16>(n, 2 * ks + h);
  // V^T fragment (A operand) through the transposing read: this lane points at row (lane%16)/4 of a
  // 4-row group and at 4 contiguous columns; it receives column 32*dt + n for the 4 rows.
  const int s16 = lane & 15;
  const int vr4 = s16 >> 2;                                   // row inside the 4-row group
  const int vcol = 16 * ((lane >> 4) & 1) + 4 * (s16 & 3);    // first of the 4 columns, inside a d-tile
  int voff[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int row = 4 * h + vr4;                              // + 32*nt + 16*s (+8): multiples of 8 keep row&3, (row>>1)&1
    voff[dt] = lds_chunk_off<NCV, Swz::Rows4>(row, 4 * dt + (vcol >> 3)) + (vcol & 7) * 2;
  }

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

  // ---- prologue ----------------------------------------------------------------------------------
  if (n_tiles > 0) {
    kdma.issue(kg, kbuf, wave_base);
    if constexpr (NSV == 2) vdma.issue(vg, vbuf, wave_base);
  }

  // One kv tile.  MASKED is set for the tiles the causal diagonal crosses; all other tiles run the
  // plain path, so the mask costs nothing where it cannot apply.
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

    // ---- S^T = K Q^T -----------------------------------------------------------------------------
    f16v sacc[RT][NT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) sacc[rt][nt] = zero16();
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const h8 kf = lds_read_h8(kcur + nt * 32 * NCK * 16 + koff[ks]);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) sacc[rt][nt] = mfma_32x32x16(kf, qf[rt][ks], sacc[rt][nt]);
      }
    }

    // ---- online softmax, one query row per lane -------------------------------------------------
    h8 pf[RT][NT][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int q_lim = q0 + wave * WM + rt * 32 + n + diag;             // last kv index this row may see
      if constexpr (MASKED) causal_mask<NT>(sacc[rt], j * Bc, q_lim, h);
      // Lazy running max: the reference point m_run of the exponent is moved (and O, l rescaled) only
      // when some row of the wave has grown past it by more than kLazyLog2 in the log2 domain.  Until
      // then P may exceed 1 by at most 2^kLazyLog2, which fp16 P and fp32 l, O absorb without loss;
      // the final O / l is unchanged because numerator and denominator share the reference point.
      const float m_tile = pair_max(lane_max<NT>(sacc[rt]));
      const bool grow = (m_tile - m_run[rt]) * c2 > kLazyLog2;          // false for -inf - -inf
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {                      // wave-uniform branch
        const float m_new = fmaxf(m_run[rt], m_tile);
        const SoftmaxStep st = softmax_step(m_run[rt], m_new, c2);
        m_run[rt] = m_new;
        l_run[rt] *= st.alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int vv = 0; vv < 16; ++vv) oacc[rt][dt][vv] *= st.alpha;
      }
      const float mc = (m_run[rt] == -INFINITY ? 0.f : m_run[rt]) * c2;
      l_run[rt] += exp_tile<NT, MASKED>(sacc[rt], c2, mc, j * Bc, q_lim, h);   // per-lane partial sum
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        pf[rt][nt][0] = pack8_rne(sacc[rt][nt], 0);
        pf[rt][nt][1] = pack8_rne(sacc[rt][nt], 8);
      }
    }

    // (B) with one buffer: V_j must have landed / K buffer must be free before K_{j+1} is fetched.
    if constexpr (NSV == 1 || NSK == 1) {
      if constexpr (NSV == 1) wait_vmcnt<0>();
      block_sync();
      if constexpr (NSK == 1) {
        if (more) kdma.issue(kg + (size_t)(j + 1) * T::kKBytes, kbuf, wave_base);
      }
    }

    // ---- O^T += V^T P^T --------------------------------------------------------------------------
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const char* vrow = vcur + (32 * nt + 16 * s) * NCV * 16;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const h4 lo = lds_read_tr_h4(vrow + voff[dt]);
          const h4 hi = lds_read_tr_h4(vrow + 8 * NCV * 16 + voff[dt]);
          const h8 vf = cat_h4(lo, hi);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) oacc[rt][dt] = mfma_32x32x16(vf, pf[rt][nt][s], oacc[rt][dt]);
        }
      }
    }
  };

  // Tiles [0, n_full) are visible to every row of the block; [n_full, n_tiles) touch the diagonal.
  int n_full = n_tiles;
  if (causal) {
    const int lim = (q0 + diag + 1) / Bc;
    n_full = lim < 0 ? 0 : (lim < n_tiles ? lim : n_tiles);
  }
  for (int j = 0; j < n_full; ++j) kv_tile(j, std::false_type{});
  for (int j = n_full; j < n_tiles; ++j) kv_tile(j, std::true_type{});

  // ---- epilogue: normalise, round, transpose through LDS, coalesced store ----------------------
  wait_vmcnt<0>();
  block_sync();                                  // every wave is done with the K/V buffers
  char* const ostage = smem + wave * WM * T::kOStride;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float l_tot = pair_sum(l_run[rt]);
    const float inv = l_tot > 0.f ? fast_rcp(l_tot) : 0.f;
    if (lse != nullptr && h == 0) {
      const size_t row = (size_t)bh * seq_q + q0 + wave * WM + rt * 32 + n;
      lse[row] = l_tot > 0.f ? m_run[rt] * softmax_scale + __logf(l_tot) : -INFINITY;
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const h2 a = pack_rne(oacc[rt][dt][4 * g] * inv, oacc[rt][dt][4 * g + 1] * inv);
        const h2 b = pack_rne(oacc[rt][dt][4 * g + 2] * inv, oacc[rt][dt][4 * g + 3] * inv);
        h4 w;
        w[0] = a[0]; w[1] = a[1]; w[2] = b[0]; w[3] = b[1];
        const int d0 = 32 * dt + 8 * g + 4 * h;
        *reinterpret_cast<h4*>(ostage + (rt * 32 + n) * T::kOStride + d0 * 2) = w;
      }
    }
  }
  wait_lgkm0();                                   // the staging region is private to this wave
  {
    half_t* og = o + ((size_t)bh * seq_q + q0 + wave * WM) * D;
    constexpr int kChunks = WM * NCV;
#pragma unroll
    for (int t = 0; t < kChunks / 64; ++t) {
      const int idx = t * 64 + lane;
      const int row = idx / NCV, c = idx % NCV;
      const u4v val = *reinterpret_cast<const u4v*>(ostage + row * T::kOStride + c * 16);
      *reinterpret_cast<u4v*>(reinterpret_cast<char*>(og) + ((size_t)row * NCV + c) * 16) = val;
    }
  }
}

}  // namespace aat
