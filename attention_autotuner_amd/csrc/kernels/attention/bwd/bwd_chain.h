// Flash-attention backward for gfx950 (MI355X).
//
// With S = scale * Q K^T, P = exp(S - lse) (lse = the forward's log-sum-exp per query row) and
// delta = rowsum(dO * O):
//     dV = P^T dO,      dP = dO V^T,      dS = P * (dP - delta),      dK = scale * dS^T Q,      dQ = scale * dS K.
// The reference declares this operator and leaves it empty (reference: python/ops/attention_interface.py:37-58,
// README.md:107); the arithmetic follows its RetNet backward (csrc/kernels/retnet/bwd/bwd_colblock.h:445-596):
// fp32 accumulation, P and dS rounded to fp16 (RNE) before the dependent contraction.
//
// Same construction as the RetNet backward of this library: no atomics, no fp32 dQ scratch.  Two
// kernels walk the (kv block, q block) pairs, each keeping its resident rows' operands in registers (a
// lane owns one resident row) and streaming the other side through LDS:
//
//     COL  resident kv rows (K, V fragments)  streams Q and dO tiles   ->  dV and dK
//     ROW  resident q rows (Q, dO fragments)  streams K and V tiles    ->  dQ
//
// A streamed tile is read both ways -- row-major b128 fragments for the first contractions
// (S^T = Q K^T resp. dP^T = dO V^T) and transposing reads for the second ones (dV^T += dO^T P,
// dK^T += Q^T dS, dQ^T += K^T dS) -- so each tile is fetched once and laid out with the dual swizzle.
// Cost: S and dP are evaluated by both kernels (7 instead of 5 contractions per score).
//
// The column kernel can also be built for one of its two outputs (OUTS): dV alone needs neither V nor dP
// (two contractions), dK alone needs everything but the dV accumulators (three).  Run as a pair they cost
// one more evaluation of S, and each fits a register budget the two-output kernel does not: two waves per
// SIMD at d = 128, and one wave per SIMD at d_qk = 256 / d_v = 512, where dV (256 accumulators per lane)
// and dK (128) cannot share a wave at all.
//
// lse2 = lse * log2(e) and delta come from attn_bwd_prepare (one pass over O and dO); the COL kernel
// copies the 2 * BY values of a streamed tile into LDS next to the tile.
#pragma once
#include <type_traits>

#include "../../utils/cdna4.h"
#include "../../utils/tile_ops.h"

#ifndef AAT_PF
#define AAT_PF 2
#endif

namespace aat {

enum class AttnBwdPass { Col, Row };

// Kd: width of q/k rows; D: width of v/o/dO rows; BX: resident rows per block; BY: rows per streamed
// tile; NS: LDS buffers of the stream (2 or 3).
template <int Kd, int D, int BX, int BY, int Nthreads, int NS, AttnBwdPass PASS>
struct AttnBwdChain {
  static constexpr bool COL = PASS == AttnBwdPass::Col;
  static constexpr int NW = Nthreads / kWave;
  static constexpr int WM = BX / NW;
  static constexpr int RT = WM / 32;
  static constexpr int NT = BY / 32;
  static constexpr int KS = Kd / 16, DS = D / 16;       // k-steps of the two first contractions
  static constexpr int KT = Kd / 32, DT = D / 32;       // output tiles of the second contractions
  static constexpr int NCK = Kd / 8, NCD = D / 8;
  static_assert(Nthreads % kWave == 0 && BX % NW == 0 && WM % 32 == 0, "each wave owns whole 32-row groups");
  static_assert(BY % 32 == 0 && Kd % 64 == 0 && D % 64 == 0, "tile shape");
  static_assert(NS == 2 || NS == 3, "buffers");
  using Y1Dma = TileDma<BY, NCK, Nthreads, Swz::Both>;  // Q (COL) or K (ROW) tile
  using Y2Dma = TileDma<BY, NCD, Nthreads, Swz::Both>;  // dO (COL) or V (ROW) tile
  static constexpr int kY1Bytes = BY * Kd * 2, kY2Bytes = BY * D * 2;
  static constexpr int kStatBytes = COL ? 1024 : 0;     // lse2 and delta of the streamed rows (2 * BY floats)
  static_assert(2 * BY * 4 <= 1024, "statistics slot");
  static constexpr int kStatInstr = COL ? (2 * BY + 63) / 64 : 0;
  static constexpr int kStageBytes = kY1Bytes + kY2Bytes + kStatBytes;
  static constexpr int kTileInstr = Y1Dma::kIters + Y2Dma::kIters + kStatInstr;   // LDS-DMA instructions per thread per tile
  static constexpr int kOCols = COL ? (D > Kd ? D : Kd) : Kd;
  static constexpr int kOStride = kOCols * 2 + 16;
  static constexpr int kMainBytes = NS * kStageBytes;
  static constexpr int kEpiBytes = BX * kOStride;
  static constexpr int kSmemBytes = kMainBytes > kEpiBytes ? kMainBytes : kEpiBytes;
};

// delta[row] = sum_d dO[row][d] * O[row][d], lse2[row] = lse[row] * log2(e); a power-of-two group of lanes per row.
template <int D> constexpr int attn_bwd_prepare_lanes_per_row() {
  return D / 8 <= 8 ? 8 : D / 8 <= 16 ? 16 : D / 8 <= 32 ? 32 : 64;
}
template <int D> constexpr int attn_bwd_prepare_rows_per_block() { return 4 * (64 / attn_bwd_prepare_lanes_per_row<D>()); }
template <int D>
__global__ void __launch_bounds__(256) attn_bwd_prepare(const half_t* __restrict__ o, const half_t* __restrict__ dO,
                                                        const float* __restrict__ lse, float* __restrict__ lse2,
                                                        float* __restrict__ delta, int rows) {
  constexpr int kChunks = D / 8;                        // 16-byte chunks per row: 8, 16, 24, 32 or 64
  constexpr int kLanesPerRow = attn_bwd_prepare_lanes_per_row<D>();   // lanes beyond the row's chunks idle
  static_assert(kChunks <= 64, "row width");
  constexpr int kRowsPerWave = 64 / kLanesPerRow;
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * 256 + threadIdx.x) >> 6;
  const int row = wave * kRowsPerWave + lane / kLanesPerRow;
  float s = 0.f;
  if (row < rows && lane % kLanesPerRow < kChunks) {
    const size_t off = (size_t)row * D + (lane % kLanesPerRow) * 8;
    const h8 a = *reinterpret_cast<const h8*>(o + off);
    const h8 b = *reinterpret_cast<const h8*>(dO + off);
#pragma unroll
    for (int i = 0; i < 8; ++i) s += (float)a[i] * (float)b[i];
  }
#pragma unroll
  for (int m = 1; m < kLanesPerRow; m <<= 1) s += __shfl_xor(s, m, 64);
  if (row < rows && lane % kLanesPerRow == 0) {
    delta[row] = s;
    lse2[row] = lse[row] * 1.4426950408889634f;
  }
}

// x1, x2: resident-side matrices (COL: k, v; ROW: q, dO); y1, y2: streamed-side matrices (COL: q, dO;
// ROW: k, v); all [B*H, S, width] fp16.  lse2, delta: [B*H, seq_q] fp32.  COL writes out1 = dV and
// out2 = dK; ROW writes out2 = dQ.  c2 = softmax_scale * log2(e); out_scale = softmax_scale.
// OUTS (COL only): 3 = both outputs, 1 = dV only (x2, delta and out2 are not touched), 2 = dK only.
template <int Kd, int D, int BX, int BY, int Nthreads, int NS, AttnBwdPass PASS, int WPE = 1, int OUTS = 3>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
attn_bwd_chain(const half_t* __restrict__ x1, const half_t* __restrict__ x2, const half_t* __restrict__ y1,
               const half_t* __restrict__ y2, const float* __restrict__ lse2, const float* __restrict__ delta,
               half_t* __restrict__ out1, half_t* __restrict__ out2, int H, int seq_k, int seq_q, float c2,
               float out_scale, int causal) {
  using T = AttnBwdChain<Kd, D, BX, BY, Nthreads, NS, PASS>;
  constexpr int RT = T::RT, NT = T::NT, KS = T::KS, DS = T::DS, KT = T::KT, DT = T::DT, NCK = T::NCK, NCD = T::NCD,
                WM = T::WM;
  constexpr int PF = AAT_PF;
  constexpr bool COL = T::COL;
  static_assert(COL ? (OUTS >= 1 && OUTS <= 3) : OUTS == 3, "output selection is a column-kernel option");
  constexpr bool kOut1 = COL && (OUTS & 1);       // dV
  constexpr bool kOut2 = !COL || (OUTS & 2);      // dK or dQ: needs dP and with it X2, delta
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int seq_x = COL ? seq_k : seq_q, seq_y = COL ? seq_q : seq_k;

  const int Tx = seq_x / BX;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  int bh = tile / Tx, xb = tile % Tx;
  if (causal) {                                   // longest blocks first: the last query blocks, the first kv blocks
    const TileId t = causal_tile(blockIdx.x, gridDim.x, Tx, !COL);
    bh = t.bh;
    xb = t.blk;
  }
  const int x0 = xb * BX;
  const int diag = seq_k - seq_q;                 // causal: score (q, kv) is kept when kv <= q + diag
  int j_begin = 0, j_end = seq_y / BY;
  if (causal) {
    if constexpr (COL) {                          // q tiles that reach kv >= x0:  q >= x0 - diag
      const int first = x0 - diag;
      j_begin = first <= 0 ? 0 : first / BY;
    } else {                                      // kv tiles with kv <= x0 + BX - 1 + diag
      const int last = x0 + BX - 1 + diag;
      const int lim = last < 0 ? 0 : last / BY + 1;
      j_end = lim < j_end ? lim : j_end;
    }
  }

  const char* y1g = reinterpret_cast<const char*>(y1 + (size_t)bh * seq_y * Kd);
  const char* y2g = reinterpret_cast<const char*>(y2 + (size_t)bh * seq_y * D);
  const float* lse_g = lse2 + (size_t)bh * seq_q;
  const float* delta_g = delta + (size_t)bh * seq_q;

  typename T::Y1Dma y1dma;
  typename T::Y2Dma y2dma;
  y1dma.init(tid);
  y2dma.init(tid);
  const int wave_base = wave * 64;

  // resident operands: this lane's row of X1 (width Kd) and of X2 (width D) as MFMA B fragments
  h8 x1f[RT][KS], x2f[RT][kOut2 ? DS : 1];
  load_q_frags<RT, KS, Kd>(x1f, x1 + ((size_t)bh * seq_x + x0 + wave * WM + n) * Kd + 8 * h);
  if constexpr (kOut2) load_q_frags<RT, DS, D>(x2f, x2 + ((size_t)bh * seq_x + x0 + wave * WM + n) * D + 8 * h);

  // LDS addresses inside stage 0: first-contraction fragments (rows n, chunk 2ks+h) and transposing reads
  uint32_t y1addr[KS], y2addr[DS], z1lo[KT], z1hi[KT], z2lo[DT], z2hi[DT];
  {
    int o1[KS], o2[DS];
    k_frag_offsets<KS, NCK, Swz::Both>(o1, n, h);
    k_frag_offsets<DS, NCD, Swz::Both>(o2, n, h);
#pragma unroll
    for (int i = 0; i < KS; ++i) y1addr[i] = lds_addr(smem + o1[i]);
#pragma unroll
    for (int i = 0; i < DS; ++i) y2addr[i] = lds_addr(smem + T::kY1Bytes + o2[i]);
    // transposing reads: rows 4h + (lane%16)/4 (+8 for the second half; the dual swizzle sees row bit 3,
    // so the second half has its own address), columns 32*tile + 16*((lane/16)%2) + 4*(lane%4) .. +3
    const int s16 = lane & 15;
    const int row = 4 * h + (s16 >> 2);
    const int col = 16 * ((lane >> 4) & 1) + 4 * (s16 & 3);
#pragma unroll
    for (int i = 0; i < KT; ++i) {
      z1lo[i] = lds_addr(smem + lds_chunk_off<NCK, Swz::Both>(row, 4 * i + (col >> 3)) + (col & 7) * 2);
      z1hi[i] = lds_addr(smem + lds_chunk_off<NCK, Swz::Both>(row + 8, 4 * i + (col >> 3)) + (col & 7) * 2);
    }
#pragma unroll
    for (int i = 0; i < DT; ++i) {
      z2lo[i] = lds_addr(smem + T::kY1Bytes + lds_chunk_off<NCD, Swz::Both>(row, 4 * i + (col >> 3)) + (col & 7) * 2);
      z2hi[i] = lds_addr(smem + T::kY1Bytes + lds_chunk_off<NCD, Swz::Both>(row + 8, 4 * i + (col >> 3)) + (col & 7) * 2);
    }
  }
  const uint32_t stat_addr = lds_addr(smem + T::kY1Bytes + T::kY2Bytes + 16 * h);   // + 32 B per register group

  // ROW: the lane's own query row statistics
  float lse_row[RT], delta_row[RT];
  if constexpr (!COL) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      lse_row[rt] = lse_g[x0 + wave * WM + rt * 32 + n];
      delta_row[rt] = delta_g[x0 + wave * WM + rt * 32 + n];
    }
  }

  // accumulators: acc1 = dV^T (COL only, D wide), acc2 = dK^T (COL) or dQ^T (ROW), Kd wide
  f16v acc1[RT][kOut1 ? DT : 1], acc2[RT][kOut2 ? KT : 1];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int i = 0; i < (kOut1 ? DT : 1); ++i) acc1[rt][i] = zero16();
#pragma unroll
    for (int i = 0; i < (kOut2 ? KT : 1); ++i) acc2[rt][i] = zero16();
  }

  // Step j of the walk works on streamed tile tile_of(j): the row kernel walks its kv tiles upwards, the column
  // kernel its query tiles downwards from the end of the sequence.  Either way the blocks of a head that run at the
  // same time start on the same tile of a causal walk and share it in L2 (a column block needs the tiles from its
  // own diagonal to the end: walked upwards every block would stream its range alone).
  const auto tile_of = [&](int j) { return COL ? j_begin + j_end - 1 - j : j; };
  auto issue = [&](int step, int st) {
    const int j = tile_of(step);
    char* base = smem + st * T::kStageBytes;
    y1dma.issue(y1g + (size_t)j * T::kY1Bytes, base, wave_base);
    y2dma.issue(y2g + (size_t)j * T::kY2Bytes, base + T::kY1Bytes, wave_base);
    if constexpr (COL) {
      // every wave copies the tile's 2*BY statistics (same bytes, same place): uniform instruction counts
#pragma unroll
      for (int i = 0; i < T::kStatInstr; ++i) {
        const int idx = i * 64 + lane;              // [0, BY): lse2, [BY, 2BY): delta
        const int c = idx < 2 * BY ? idx : 2 * BY - 1;
        const float* src = c < BY ? lse_g + j * BY + c : delta_g + j * BY + (c - BY);
        __builtin_amdgcn_global_load_lds((const AAT_AS1 void*)(uintptr_t)src,
                                         (AAT_AS3 void*)(base + T::kY1Bytes + T::kY2Bytes + i * 256), 4, 0, 0);
      }
    }
  };
  if (j_begin < j_end) {
    issue(j_begin, 0);
    if constexpr (NS == 3) {
      if (j_begin + 1 < j_end) issue(j_begin + 1, 1);
    }
  }

  auto y_tile = [&](const int j, auto st_tag) {
    constexpr int st = decltype(st_tag)::value;
    constexpr int off = st * T::kStageBytes;
    const bool more = (j + 1 < j_end);
    if constexpr (WPE == 1) {
      // one wave per SIMD: outputs in the accumulation registers, resident fragments in vector registers
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if constexpr (kOut1) {
#pragma unroll
          for (int i = 0; i < DT; ++i) asm volatile("" : "+a"(acc1[rt][i]));
        }
        if constexpr (kOut2) {
#pragma unroll
          for (int i = 0; i < KT; ++i) asm volatile("" : "+a"(acc2[rt][i]));
#pragma unroll
          for (int i = 0; i < DS; ++i) asm volatile("" : "+v"(x2f[rt][i]));
        }
#pragma unroll
        for (int i = 0; i < KS; ++i) asm volatile("" : "+v"(x1f[rt][i]));
      }
    }
    // tile j has landed (with three buffers tile j+1 may still be in flight); every wave is past tile j-1
    if constexpr (NS == 3) {
      if (more) wait_vmcnt<T::kTileInstr>();
      else wait_vmcnt<0>();
    } else {
      wait_vmcnt<0>();
    }
    block_sync();
    if constexpr (NS == 3) {
      if (j + 2 < j_end) issue(j + 2, (st + 2) % 3);
    } else {
      if (more) issue(j + 1, st ^ 1);
    }

    // first contractions: s = Y1 X1^T (scores), p = Y2 X2^T (dP), both transposed (lane owns resident row)
    // the score tiles accumulate in vector registers when the outputs alone fill the accumulation registers
    // ... and also when they fit next to the resident fragments anyway: a score tile in accumulation registers is
    // read back one register at a time for the element-wise step (64 v_accvgpr_read per 64-row tile at d 128;
    // -0.7 ... -1.0 % on the whole backward, same bits)
    constexpr bool kFitsVec = RT * (KS + (kOut2 ? DS : 0)) * 4 + RT * NT * 32 + 72 <= 208;
    constexpr bool kVacc = WPE == 1 && (kFitsVec || RT * ((kOut1 ? DT : 0) + (kOut2 ? KT + NT : 0) + NT) * 16 > 256);
    f16v s[RT][NT], dp[RT][kOut2 ? NT : 1];
    qk_gemm_steps<RT, NT, KS, NCK, PF, kVacc>(s, x1f, y1addr, off, [](int) {});
    if constexpr (kOut2) qk_gemm_steps<RT, NT, DS, NCD, PF, kVacc>(dp, x2f, y2addr, off, [](int) {});

    // P = exp2(s*c2 - lse2[q]),  dS = P * (dP - delta[q]);  register v of tile t is streamed row 32t + 8(v/4) + 4h + v%4.
    // Only a tile the diagonal crosses runs the masking code.  COL: the statistics of the streamed rows come
    // from LDS four rows at a time, read by hand one group ahead (a tracked read here is answered with a
    // full lgkmcnt(0) per group: eight exposed LDS round trips per tile for the only wave of the SIMD).
    const int jt = tile_of(j);                      // the tile of this step
    const bool diag_tile = causal && (COL ? (x0 + BX - 1 > jt * BY + diag) : ((jt + 1) * BY - 1 > x0 + diag));
    auto softmax_part = [&](auto masked_tag) {
      constexpr bool MASKED = decltype(masked_tag)::value;
      constexpr int G = RT * NT * 4;                                 // groups of four streamed rows
      f4v l2r[2], dlr[2];
      auto read_stats = [&](auto it) {
        constexpr int i = decltype(it)::value, tg = i % (NT * 4);    // the statistics do not depend on rt
        l2r[i % 2] = lds_read_f4_async(stat_addr, off + (32 * (tg / 4) + 8 * (tg % 4)) * 4);
        if constexpr (kOut2) dlr[i % 2] = lds_read_f4_async(stat_addr, off + (BY + 32 * (tg / 4) + 8 * (tg % 4)) * 4);
      };
      if constexpr (COL) read_stats(std::integral_constant<int, 0>{});
      static_for<G>([&](auto it) {
        constexpr int i = decltype(it)::value, rt = i / (NT * 4), t = (i / 4) % NT, g = i % 4;
        if constexpr (COL) {                     // the next group's read goes into the other slot; wait on this slot before taking its value
          if constexpr (i + 1 < G) {
            read_stats(std::integral_constant<int, i + 1>{});
            if constexpr (kOut2) lds_wait_younger<2>(l2r[i % 2], dlr[i % 2]);
            else lds_wait_younger<1>(l2r[i % 2]);
          } else {
            if constexpr (kOut2) lds_wait_younger<0>(l2r[i % 2], dlr[i % 2]);
            else lds_wait_younger<0>(l2r[i % 2]);
          }
        }
        f4v l2 = l2r[i % 2], dl = {0.f, 0.f, 0.f, 0.f};
        if constexpr (kOut2) dl = dlr[i % 2];
        // The score of resident row x and streamed row y = jt*BY + c + 4h (c = 32t + 8g + e, a constant) is masked
        // when kv > q + diag: COL (x is kv) x - diag - jt*BY - 4h > c, ROW (x is q) c > x + diag - jt*BY - 4h.
        const int xrow = x0 + wave * WM + rt * 32 + n;               // resident row of this lane
        const int lim = (COL ? xrow - diag : xrow + diag) - jt * BY - 4 * h;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          constexpr int vbase = 4 * g, cbase = 32 * t + 8 * g;
          const int v = vbase + e;
          const float lrow = COL ? l2[e] : lse_row[rt];
          float p = fast_exp2(s[rt][t][v] * c2 - lrow);
          if constexpr (MASKED) {
            if (COL ? lim > cbase + e : cbase + e > lim) p = 0.f;
          }
          s[rt][t][v] = p;
          if constexpr (kOut2) {
            const float drow = COL ? dl[e] : delta_row[rt];
            dp[rt][t][v] = p * (dp[rt][t][v] - drow);
          }
        }
      });
    };
    if (diag_tile) softmax_part(std::true_type{});
    else softmax_part(std::false_type{});

    // second contractions: COL  dV^T += dO^T P  and  dK^T += Q^T dS;   ROW  dQ^T += K^T dS
    h8 ef[RT][NT][2];
    if constexpr (kOut1) {
      pv_gemm_steps_hl<RT, NT, DT, NCD, PF>(acc1, ef, z2lo, z2hi, off, [&](int g) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) ef[rt][g >> 1][g & 1] = pack8_rne(s[rt][g >> 1], 8 * (g & 1));
      });
    }
    if constexpr (kOut2) {
      pv_gemm_steps_hl<RT, NT, KT, NCK, PF>(acc2, ef, z1lo, z1hi, off, [&](int g) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) ef[rt][g >> 1][g & 1] = pack8_rne(dp[rt][g >> 1], 8 * (g & 1));
      });
    }
  };
  for (int j = j_begin; j < j_end; j += NS) {
    static_for<NS>([&](auto k_tag) {
      constexpr int k = decltype(k_tag)::value;
      if (k == 0 || j + k < j_end) y_tile(j + k, std::integral_constant<int, k>{});
    });
  }

  // ---- epilogue: scale, round, transpose through wave-private LDS, 16-byte stores ---------------------
  wait_vmcnt<0>();
  block_sync();
  char* const ostage = smem + wave * WM * T::kOStride;
  auto store = [&](auto& acc, auto cols_tag, half_t* out, float sc) {
    constexpr int W = decltype(cols_tag)::value;           // output row width
    constexpr int NTILE = W / 32, kChunksPerRow = W / 8;
    half_t* og = out + ((size_t)bh * seq_x + x0 + wave * WM) * W;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int dt = 0; dt < NTILE; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const h2 a = pack_rne(acc[rt][dt][4 * g] * sc, acc[rt][dt][4 * g + 1] * sc);
          const h2 b = pack_rne(acc[rt][dt][4 * g + 2] * sc, acc[rt][dt][4 * g + 3] * sc);
          h4 w;
          w[0] = a[0]; w[1] = a[1]; w[2] = b[0]; w[3] = b[1];
          *reinterpret_cast<h4*>(ostage + (rt * 32 + n) * T::kOStride + (32 * dt + 8 * g + 4 * h) * 2) = w;
        }
    wait_lgkm0();
    constexpr int kChunks = WM * kChunksPerRow;
#pragma unroll
    for (int t = 0; t < kChunks / 64; ++t) {
      const int idx = t * 64 + lane;
      const int row = idx / kChunksPerRow, c = idx % kChunksPerRow;
      const u4v val = *reinterpret_cast<const u4v*>(ostage + row * T::kOStride + c * 16);
      *reinterpret_cast<u4v*>(reinterpret_cast<char*>(og) + (size_t)row * W * 2 + c * 16) = val;
    }
    wait_lgkm0();                                           // the staging rows are reused by the next output
  };
  if constexpr (kOut1) store(acc1, std::integral_constant<int, D>{}, out1, 1.0f);
  if constexpr (kOut2) store(acc2, std::integral_constant<int, Kd>{}, out2, out_scale);
}

}  // namespace aat
