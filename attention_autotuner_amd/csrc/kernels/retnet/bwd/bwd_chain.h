// RetNet parallel retention backward for gfx950 (MI355X).
//
// With r held constant (the reference detaches it), P = (Q K^T * M) / r and
//     dV = P^T dO,      dS = (dO V^T / r) * M,      dK = dS^T Q,      dQ = dS K,
// P and dS rounded to fp16 before the dependent contraction, fp32 accumulation -- the arithmetic of
// the reference's column-block kernel (reference: csrc/kernels/retnet/bwd/bwd_colblock.h:445-596, closed
// forms at :522-576, fp16 rounding at :509 and :551).
//
// The reference walks (kv block, q block) pairs once, keeps dK and dV in registers and pushes dQ
// through fp32 atomics into scratch that a second kernel converts (convert_dq, :742-811).  On MI355X
// the atomic traffic (S_q*S_kv/Bc*Kd*4 bytes per head) costs more than the arithmetic it saves and
// dK + dV do not fit one wave's registers at d_qk=256, d_v=512.  Each gradient is instead its own pass
// of one "chained contraction" kernel, the same shape as the forward kernel:
//
//     T^T[y][x] = sum_k Y[y][k] X[x][k]      X: block-resident rows (a lane owns one), Y: streamed tiles
//     E[y][x]   = half( T * M / r )
//     Out[x][:] = sum_y E[y][x] Z[y][:]      Z: streamed tiles, read transposed
//
//     pass      X    Y    Z    Out   lane owns   r index   mask access
//     dV  COL   K    Q    dO   dV    kv row      y (q)     transposed (ds_read_b64_tr_b16)
//     dK  COL   V    dO   Q    dK    kv row      y (q)     transposed
//     dQ  ROW   dO   V    K    dQ    q row       x (q)     row-major
//
// No atomics, no scratch, deterministic; dQ is written directly in fp16, so the reference's second
// kernel has no counterpart.  Cost: dO V^T is evaluated twice (3*(d_qk+d_v) instead of 3*d_qk+2*d_v
// multiply-adds per score) and, for an output wider than DZB columns, the first contraction is repeated
// per column slice (grid.y slices).
#pragma once
#include <type_traits>

#include "../../utils/acc_file.h"
#include "../../utils/cdna4.h"
#include "../../utils/mask_extents.h"
#include "../../utils/retention.h"
#include "../../utils/tile_ops.h"
#include "ds_layout.h"

#ifndef AAT_PF
#define AAT_PF 4
#endif

namespace aat {

enum class BwdPass { Col, Row };

// KX: contraction width of the first product (columns of X and Y); DZ: columns of Z and Out;
// DZB: output columns handled by one block (DZ / DZB blocks along grid.y);
// BX: resident rows per block; BY: rows per streamed tile; NSY / NSZ: LDS buffers of the Y(+mask) and Z streams.
template <int KX, int DZ, int DZB, int BX, int BY, int Nthreads, int NSY, int NSZ, BwdPass PASS>
struct RetBwdChain {
  static constexpr int NW = Nthreads / kWave;
  static constexpr int WM = BX / NW;
  static constexpr int RT = WM / 32;
  static constexpr int NT = BY / 32;
  static constexpr int KS = KX / 16;
  static constexpr int DT = DZB / 32;
  static constexpr int NCY = KX / 8, NCZ = DZB / 8;
  // mask tile: rows = q, columns = kv.  COL: q is the streamed index (BY rows x BX columns); ROW: BX rows x BY columns.
  static constexpr int kMRows = PASS == BwdPass::Col ? BY : BX;
  static constexpr int kMCols = PASS == BwdPass::Col ? BX : BY;
  static constexpr int NCM = kMCols / 8;
  static_assert(Nthreads % kWave == 0 && BX % NW == 0 && WM % 32 == 0, "each wave owns whole 32-row groups");
  static_assert(BY % 32 == 0 && KX % 64 == 0 && DZ % DZB == 0 && DZB % 64 == 0, "tile shape");
  static_assert(NSY >= 1 && NSY <= 3 && (NSZ == 1 || NSZ == 2) && (NSY < 3 || NSZ == 2), "buffers");
  using YDma = TileDma<BY, NCY, Nthreads, Swz::Rows16>;
  using ZDma = TileDma<BY, NCZ, Nthreads, Swz::Rows4>;
  using MDma = TileDma<kMRows, NCM, Nthreads, PASS == BwdPass::Col ? Swz::Rows4 : Swz::Rows16>;
  static constexpr int kYBytes = BY * KX * 2, kZBytes = BY * DZB * 2, kMBytes = kMRows * kMCols * 2;
  static constexpr int kOStride = DZB * 2 + 16;
  static constexpr int kMainBytes = NSY * (kYBytes + kMBytes) + NSZ * kZBytes;
  static constexpr int kEpiBytes = BX * kOStride;
  static constexpr int kSmemBytes = kMainBytes > kEpiBytes ? kMainBytes : kEpiBytes;
  // DS_OUT variant of the row pass: a wave-private staging area behind the stream buffers, in which a dS tile
  // turns from 8-byte pieces per lane into whole rows
  static constexpr int kDsStride = BY * 2 + 16;
  static constexpr int kDsStageBytes = BX * kDsStride;
  static constexpr int kSmemBytesDsOut = (kMainBytes + kDsStageBytes > kEpiBytes) ? kMainBytes + kDsStageBytes : kEpiBytes;
};

// x, y, z, out: [B*H, S, width] fp16 with S = seq_x for x/out and seq_y for y/z; mask [H, seq_q, seq_k];
// r [B*H, seq_q].  For COL passes seq_x = seq_k, seq_y = seq_q; for the ROW pass the other way round.
// `causal` promises mask == 0 above the diagonal and only shortens the walk over streamed tiles.
// DECAY: the mask is gamma_h^(q + diag - kv) below the diagonal and zero above it, built in registers
// from lg2gamma[h] = log2(gamma_h); `mask` is not read and tiles above the diagonal are skipped.
// DS_OUT (row pass only): the fp16 E tiles (= dS) this pass forms are also written to ds_out (64 x 64 blocks, ds_layout.h), for
// a dK kernel that reads them instead of evaluating them again (dk_from_ds.h).  Only the tiles of the walk are written.
template <int KX, int DZ, int DZB, int BX, int BY, int Nthreads, int NSY, int NSZ, BwdPass PASS, int WPE = 1,
          bool DECAY = false, bool DS_OUT = false>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
ret_bwd_chain(const half_t* __restrict__ x, const half_t* __restrict__ y, const half_t* __restrict__ z,
              const half_t* __restrict__ mask, const float* __restrict__ r, half_t* __restrict__ out, int H,
              int seq_k, int seq_q, int causal, const float* __restrict__ lg2gamma = nullptr,
              const int* __restrict__ extents = nullptr, half_t* __restrict__ ds_out = nullptr) {
  static_assert(!DS_OUT || PASS == BwdPass::Row, "dS is written by the row pass");
  using T = RetBwdChain<KX, DZ, DZB, BX, BY, Nthreads, NSY, NSZ, PASS>;
  constexpr int RT = T::RT, NT = T::NT, KS = T::KS, DT = T::DT, NCY = T::NCY, NCZ = T::NCZ, NCM = T::NCM, WM = T::WM;
  // An output tile that fills the accumulation file (one wave per SIMD, 32 rows x 512 columns: the dV pass at d_v 512)
  // lives there by number, outside the compiler's allocation (utils/acc_file.h): with the tile as a C++ value the
  // variants with more than one buffer per stream -- one loop body per ring slot -- come out with the sixteen tuples
  // placed differently from body to body and hundreds of bytes of scratch traffic per tile to reconcile them.
  // (One row group per wave only: with two the resident fragments and the score tile no longer fit 256 vector registers,
  // the compiler would reach for the accumulation file itself, and the build would be rejected.)
  constexpr bool kNumbered = WPE == 1 && RT == 1 && DT * 16 == 256;
  if constexpr (kNumbered) acc_claim_all();
  if constexpr (DECAY) causal = 1;
  constexpr int PF = AAT_PF;
  constexpr bool COL = PASS == BwdPass::Col;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* const ybuf = smem;
  char* const mbuf = smem + NSY * T::kYBytes;
  char* const zbuf = mbuf + NSY * T::kMBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int seq_x = COL ? seq_k : seq_q, seq_y = COL ? seq_q : seq_k;

  const int Tx = seq_x / BX;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  int bh = tile / Tx, xb = tile % Tx;
  if (causal || extents != nullptr) {             // longest blocks first: the last query blocks, the first kv blocks
    const TileId t = causal_tile(blockIdx.x, gridDim.x, Tx, !COL);
    bh = t.bh;
    xb = t.blk;
  }
  const int x0 = xb * BX;
  const int dz0 = blockIdx.y * DZB;               // first output column of this block
  const int diag = seq_k - seq_q;                 // mask[q][kv] may be non-zero only for kv <= q + diag
  int j_begin = 0, j_end = seq_y / BY;
  if (extents != nullptr) {                       // the streamed tiles in which the mask has a non-zero entry for these rows
    const MaskExtents e = mask_extents_at(extents, H, seq_q, seq_k);
    int lo, hi;
    if constexpr (COL) mask_col_range(e, bh % H, seq_q, seq_k, x0, BX, lo, hi);
    else mask_row_range(e, bh % H, seq_q, x0, BX, lo, hi);
    mask_tile_range(lo, hi, BY, j_end, j_begin, j_end);
  } else if (causal) {
    if constexpr (COL) {                          // q tiles that reach kv >= x0:  q >= x0 - diag
      const int first = x0 - diag;
      j_begin = first <= 0 ? 0 : first / BY;
    } else {                                      // kv tiles with kv <= x0 + BX - 1 + diag
      const int last = x0 + BX - 1 + diag;
      const int lim = last < 0 ? 0 : last / BY + 1;
      j_end = lim < j_end ? lim : j_end;
    }
  }

  const char* yg = reinterpret_cast<const char*>(y + (size_t)bh * seq_y * KX);
  const char* zg = reinterpret_cast<const char*>(z + ((size_t)bh * seq_y) * DZ + dz0);
  // mask tile origin: COL -> rows = streamed q, columns = resident kv;  ROW -> rows = resident q, columns = streamed kv
  const half_t* mhead = DECAY ? nullptr : mask + (size_t)(bh % H) * seq_q * seq_k;
  const char* mg = DECAY ? nullptr : reinterpret_cast<const char*>(COL ? mhead + x0 : mhead + (size_t)x0 * seq_k);
  DecayMask<NT, !COL> decay;
  if constexpr (DECAY) decay.init(lg2gamma[bh % H], h);

  typename T::YDma ydma;
  typename T::ZDma zdma;
  typename T::MDma mdma;
  ydma.init(tid);
  zdma.init(tid, DZ * 2);
  mdma.init(tid, seq_k * 2);
  const int wave_base = wave * 64;

  h8 xf[RT][KS];
  load_q_frags<RT, KS, KX>(xf, x + ((size_t)bh * seq_x + x0 + wave * WM + n) * KX + 8 * h);
  uint32_t yaddr[KS], zaddr[DT], maddr[RT][NT * 4];
  {
    int yoff[KS], zoff[DT];
    k_frag_offsets<KS, NCY>(yoff, n, h);
    v_frag_offsets<DT, NCZ>(zoff, lane);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) yaddr[ks] = lds_addr(ybuf + yoff[ks]);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) zaddr[dt] = lds_addr(zbuf + zoff[dt]);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < NT * 4; ++i) {
        if constexpr (COL) {
          // transposing read: score tile t = i/4, register group g = i%4 -> q rows 32t + 8g + 4h + (lane%16)/4,
          // kv columns wave*WM + 32rt + 16*((lane/16)%2) + 4*(lane%4) .. +3; this lane receives column n.
          const int s16 = lane & 15;
          const int row = 32 * (i >> 2) + 8 * (i & 3) + 4 * h + (s16 >> 2);
          const int col = wave * WM + rt * 32 + 16 * ((lane >> 4) & 1) + 4 * (s16 & 3);
          maddr[rt][i] = lds_addr(mbuf + lds_chunk_off<NCM, Swz::Rows4>(row, col >> 3) + (col & 7) * 2);
        } else {
          maddr[rt][i] = lds_addr(mbuf + lds_chunk_off<NCM, Swz::Rows16>(wave * WM + rt * 32 + n, i) + 8 * h);
        }
      }
  }
  float inv_r_row[RT];                            // ROW pass: 1/r of the lane's own query row
  if constexpr (!COL) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) inv_r_row[rt] = fast_rcp(r[(size_t)bh * seq_q + x0 + wave * WM + rt * 32 + n]);
  }
  const float* rg = r + (size_t)bh * seq_q;       // COL pass: r of the streamed query rows

  f16v acc[RT][DT];                               // unused when the tile lives in numbered registers
  if constexpr (kNumbered) {
    acc_zero<0, 256>();
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[rt][dt] = zero16();
  }

  // Streamed tiles travel through rings of NSY (Y + mask) and NSZ (Z) LDS buffers; `st` is a ring slot.
  // Step j of the walk (j_begin <= j < j_end) works on streamed tile tile_of(j).  A row pass walks its kv tiles
  // upwards: in a causal walk every query block starts at kv tile 0, so the blocks of a head that run at the same
  // time read the same tiles at the same time and all but the first read hit L2.  A column pass needs the query
  // tiles from its own diagonal to the END of the sequence; walking them downwards from the end gives its blocks
  // the same common start (walking upwards each block streams its range alone and the pass draws 600 - 780 MB
  // through L2 misses for 100 MB of tensors).  Every mask mode walks in this order, so all of them keep giving
  // the same bits.
  const auto tile_of = [&](int j) { return COL ? j_begin + j_end - 1 - j : j; };
  auto issue_ym = [&](int j, int st) {            // Y tile and mask tile of step j travel together
    const int jt = tile_of(j);
    ydma.issue(yg + (size_t)jt * T::kYBytes, ybuf + st * T::kYBytes, wave_base);
    if constexpr (!DECAY) {
      const char* msrc = COL ? mg + (size_t)jt * BY * seq_k * 2 : mg + (size_t)jt * BY * 2;
      mdma.issue(msrc, mbuf + st * T::kMBytes, wave_base);
    }
  };
  auto issue_z = [&](int j, int st) {
    zdma.issue(zg + (size_t)tile_of(j) * BY * DZ * 2, zbuf + st * T::kZBytes, wave_base);
  };
  auto load_r = [&](f4v (&rv)[COL ? NT * 4 : 1], int j) {   // COL pass: r of the step's query rows, as this lane sees them
    if constexpr (COL) {
      const int jt = tile_of(j);
#pragma unroll
      for (int i = 0; i < NT * 4; ++i)
        rv[i] = *reinterpret_cast<const f4v*>(rg + jt * BY + 32 * (i >> 2) + 8 * (i & 3) + 4 * h);
    }
  };
  constexpr int kYmInstr = T::YDma::kIters + (DECAY ? 0 : T::MDma::kIters);   // LDS-DMA instructions per thread for one Y (+ mask) tile
  constexpr int kRInstr = COL ? NT * 4 : 0;                     // register loads of r per tile
  constexpr int kDsInstr = DS_OUT ? RT * BY / 16 : 0;           // 16-byte stores of the dS tile per lane, the youngest memory operations of a tile
  // Issue order (three Y/mask buffers):  prologue  YM(j0) Z(j0) YM(j0+1);  tile j  Z(j+1) YM(j+2).
  // Loads retire in order, so "at most kYmInstr (+ the r loads of the next tile) outstanding" at the top
  // of tile j means YM(j) and Z(j) have landed while YM(j+1) may still be in flight: a Y/mask tile gets
  // two tile times to arrive, a Z tile one.  With one or two buffers every wait drains the queue.
  if (j_begin < j_end) {
    issue_ym(j_begin, 0);
    if constexpr (NSZ == 2) issue_z(j_begin, 0);
    if constexpr (NSY == 3) {
      if (j_begin + 1 < j_end) issue_ym(j_begin + 1, 1);
    }
  }
  f4v rv[COL ? NT * 4 : 1];
  if (j_begin < j_end) load_r(rv, j_begin);

  // One tile, with its ring slots as compile-time constants so every LDS offset folds into an immediate;
  // the walk below repeats with period lcm(NSY, NSZ).
  auto y_tile = [&](const int j, auto ys_tag, auto zs_tag) {
    constexpr int ys = decltype(ys_tag)::value, zs = decltype(zs_tag)::value;
    constexpr int ys1 = (ys + 1) % NSY, ys2 = (ys + 2) % NSY, zs1 = (zs + 1) % NSZ;
    const bool more = (j + 1 < j_end);
    if constexpr (WPE == 1) {
      // Above 256 registers the file is split into 256 vector and 256 accumulation registers.  Pin the
      // output accumulators to the accumulation half and the resident fragments to the vector half at
      // every tile boundary; left alone the allocator parks the fragments in accumulation registers and
      // copies four of them back in front of every MFMA.
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if constexpr (!kNumbered) {
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) asm volatile("" : "+a"(acc[rt][dt]));
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xf[rt][ks]));
      }
    }
    f4v rv_next[COL ? NT * 4 : 1];                // r of the next tile's rows: a full tile time to arrive
    if (more) load_r(rv_next, j + 1);
    sched_fence();
    // (A) Y_j and mask_j (and with two Z buffers Z_j) have landed; every wave is past the previous tile.
    if constexpr (NSY == 3) {
      if (more) wait_vmcnt<kYmInstr + kRInstr + kDsInstr>();
      else wait_vmcnt<0>();
    } else {
      // the previous tile's dS stores are the youngest memory operations in flight and nobody waits for them
      if (DS_OUT && j > j_begin) wait_vmcnt<kDsInstr>();
      else wait_vmcnt<0>();
    }
    block_sync();
    // The copies this tile starts -- Z_j (one Z buffer) or Z_{j+1} (two), then Y/mask_{j+1} (two Y buffers) or
    // Y/mask_{j+2} (three) -- go out one LDS-DMA instruction per step of the first contraction: issued in a
    // burst each of them holds the only wave of the SIMD for 100 cycles and more, between matrix
    // instructions for about half of that.  The order (Z before Y/mask) is the one the waits above count on.
    constexpr int kZi = T::ZDma::kIters, kYi = T::YDma::kIters, kMi = DECAY ? 0 : T::MDma::kIters;
    const bool z_now = NSZ == 1 || more;
    const bool ym_now = NSY == 3 ? (j + 2 < j_end) : (NSY == 2 && more);
    const int zj = tile_of(NSZ == 1 ? j : j + 1), yj = tile_of(NSY == 3 ? j + 2 : j + 1);   // tiles, not steps
    const int jt = tile_of(j);
    constexpr int zslot = NSZ == 1 ? 0 : zs1, yslot = NSY == 3 ? ys2 : ys1;
    const char* const zsrc = zg + (size_t)zj * BY * DZ * 2;
    const char* const ysrc = yg + (size_t)yj * T::kYBytes;
    const char* const msrc = DECAY ? nullptr : (COL ? mg + (size_t)yj * BY * seq_k * 2 : mg + (size_t)yj * BY * 2);
    auto issue_nth = [&](int i) {
      if (i < kZi) {
        if (z_now) zdma.issue_one(i, zsrc, zbuf + zslot * T::kZBytes, wave_base);
      } else if (i < kZi + kYi) {
        if (NSY > 1 && ym_now) ydma.issue_one(i - kZi, ysrc, ybuf + yslot * T::kYBytes, wave_base);
      } else if (i < kZi + kYi + kMi) {
        if constexpr (!DECAY) {
          if (NSY > 1 && ym_now) mdma.issue_one(i - kZi - kYi, msrc, mbuf + yslot * T::kMBytes, wave_base);
        }
      }
    };
    constexpr int yoff = ys * T::kYBytes, moff = ys * T::kMBytes, zoff = zs * T::kZBytes;

    f16v tacc[RT][NT];
    // the score tile accumulates in vector registers when the outputs fill the accumulation registers
    constexpr bool kVacc = WPE == 1 && RT * (DT + NT) * 16 > 256;
    // COL: r of this tile's query rows turns into 1/r here, a reciprocal per step, in the shadow of the matrix
    // instructions (16 of them in a row cost 140 cycles in front of the element-wise step)
    qk_gemm_steps<RT, NT, KS, NCY, PF, kVacc>(tacc, xf, yaddr, yoff, [&](int step) {
      issue_nth(step);
      if constexpr (COL) {
        constexpr int kFirst = NT * KS > 2 * NT * 16 ? NT * KS - NT * 16 : 0;      // late: the loads have landed long ago
        if (step >= kFirst && step - kFirst < NT * 16) {
          const int i = step - kFirst;
          rv[i >> 2][i & 3] = fast_rcp(rv[i >> 2][i & 3]);
        }
      }
    });
    if constexpr (COL && NT * KS < NT * 16) {       // fewer steps than values: the rest here
#pragma unroll
      for (int i = NT * KS; i < NT * 16; ++i) rv[i >> 2][i & 3] = fast_rcp(rv[i >> 2][i & 3]);
    }
    static_for<(kZi + kYi + kMi > NT * KS ? kZi + kYi + kMi - NT * KS : 0)>([&](auto t) {
      issue_nth(NT * KS + decltype(t)::value);      // more copies than steps: the rest in one go
    });
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if constexpr (DECAY) {
        // this lane's resident index, shifted so that the exponent is (streamed origin) -/+ own
        const int xrow0 = x0 + wave * WM + rt * 32;
        if constexpr (COL) {                       // lane owns kv = xrow0 + n; registers run over q rows j*BY + off
          const int base = jt * BY - (xrow0 + n - diag);
          const auto inv_r = [&](int t, int v) { return rv[4 * t + (v >> 2)][v & 3]; };
          if (jt * BY < xrow0 + 31 - diag) decay.template apply<true>(tacc[rt], base, inv_r);
          else decay.template apply<false>(tacc[rt], base, inv_r);
        } else {                                   // lane owns q = xrow0 + n; registers run over kv columns j*BY + off
          const int base = xrow0 + n + diag - jt * BY;
          const float ir = inv_r_row[rt];
          const auto inv_r = [&](int, int) { return ir; };
          if ((jt + 1) * BY - 1 > xrow0 + diag) decay.template apply<true>(tacc[rt], base, inv_r);
          else decay.template apply<false>(tacc[rt], base, inv_r);
        }
      } else if constexpr (COL) {
#pragma unroll
        for (int i = 0; i < NT * 4; ++i) {
          const h4 m = lds_read_tr_h4_at(maddr[rt][i] + moff);
#pragma unroll
          for (int e = 0; e < 4; ++e)
            tacc[rt][i >> 2][4 * (i & 3) + e] *= (float)m[e] * rv[i][e];
        }
      } else {
        apply_mask<NT>(tacc[rt], maddr[rt], moff);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int vv = 0; vv < 16; ++vv) tacc[rt][t][vv] *= inv_r_row[rt];
      }
    }

    // (B) with one buffer: Z_j must have landed / Y and mask buffers must be free before the next fetch.
    if constexpr (NSZ == 1 || NSY == 1) {
      if constexpr (NSZ == 1) wait_vmcnt<0>();
      block_sync();
    }
    // DS_OUT: the tile as the second contraction will see it (the same roundings).  A lane holds 8-byte pieces of its
    // row (kv 8g + 4h .. + 3): stored as they are, every instruction touches 32 rows 16 bytes at a time and the pass
    // runs a third longer.  Through a wave-private staging area they leave as whole rows, 16 bytes per lane.  The three
    // steps -- into the staging area, back out of it, to memory -- ride along with successive groups of the second
    // contraction, so the latency of each passes under matrix instructions; LDS executes a wave's instructions in
    // order, so the reads need no wait for the writes.  The LDS accesses are written as instructions: in front of an
    // LDS access it can see, the compiler waits for every LDS-DMA copy in flight, here the next tile's.
    constexpr int kChunksPerRow = BY / 8, kRowsPerInstr = 64 / kChunksPerRow, kStores = DS_OUT ? WM * kChunksPerRow / 64 : 1;
    static_assert(!DS_OUT || (64 % kChunksPerRow == 0 && WM <= 64), "whole rows per store instruction, in one row of dS blocks");
    static_assert(!DS_OUT || kStores <= 8, "reads of the staging area in flight");
    char* const stage = smem + T::kMainBytes + wave * WM * T::kDsStride;
    f4v staged[kStores];
    // The two lanes of a row hold alternate 8-byte pieces of it (kv 8g + 4h .. + 3).  Written as they are, the 32 rows
    // of an instruction land 36 banks apart and collide four at a time.  The lanes first trade pieces (one
    // v_permlane32_swap per register: the lower lane gives its piece of group 2k+1 for the upper lane's piece of
    // group 2k), so each holds 16 contiguous bytes, kv 16k + 8h .. + 7, and writes them with one conflict-free
    // 16-byte instruction: half the LDS writes, no conflicts, two swaps per write.
    const auto ds_stage = [&]() {
      const uint32_t st_w = lds_addr(stage + n * T::kDsStride + 16 * h);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int k2 = 0; k2 < 2; ++k2) {
            uint32_t lo[2], hi[2];                       // the pieces of groups 2k and 2k+1, two halfs per register
#pragma unroll
            for (int i = 0; i < 2; ++i) {
              const h2 a = pack_rne(tacc[rt][t][8 * k2 + 2 * i], tacc[rt][t][8 * k2 + 2 * i + 1]);
              const h2 b = pack_rne(tacc[rt][t][8 * k2 + 4 + 2 * i], tacc[rt][t][8 * k2 + 4 + 2 * i + 1]);
              __builtin_memcpy(&lo[i], &a, 4);
              __builtin_memcpy(&hi[i], &b, 4);
            }
            u4v w;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
              // result[0]: {lower lanes keep lo, upper lanes get the lower lanes' hi}; result[1]: {lower lanes get the
              // upper lanes' lo, upper lanes keep hi}
              const u2v sw = __builtin_amdgcn_permlane32_swap(lo[i], hi[i], false, false);
              w[i] = sw[0];
              w[2 + i] = sw[1];
            }
            asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(st_w), "v"(w), "i"(rt * 32 * T::kDsStride + (32 * t + 16 * k2) * 2));
          }
    };
    const auto ds_fetch = [&]() {
      const uint32_t st_r = lds_addr(stage + (lane / kChunksPerRow) * T::kDsStride + (lane % kChunksPerRow) * 16);
#pragma unroll
      for (int i = 0; i < kStores; ++i) staged[i] = lds_read_f4_async(st_r, i * kRowsPerInstr * T::kDsStride);
    };
    const auto ds_store = [&]() {
      half_t* const dst = ds_out + ds_block_offset(bh, x0 + wave * WM + lane / kChunksPerRow, jt * BY + (lane % kChunksPerRow) * 8, seq_q, seq_k);
      static_for<kStores>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        lds_wait_younger<kStores - 1 - i>(staged[i]);
        // rows of one store instruction lie in one 64-row block (kRowsPerInstr divides 64): 64 elements apart
        __builtin_nontemporal_store(staged[i], reinterpret_cast<f4v*>(dst + (size_t)i * kRowsPerInstr * 64));
      });
    };
    // What this tile sends to memory from here -- with one Y buffer the copy of the next Y and mask tile, with DS_OUT
    // the dS tile -- goes out behind the first operand reads of the second contraction.  Where those reads are left
    // to the compiler (more than one wave per SIMD) it waits in front of the first of them for the Z copy with
    // vmcnt(0), since it cannot see the wait above, and that would take in everything issued before the read too.
    constexpr int G = NT * 2;                       // groups of the second contraction
    const auto ride_along = [&](int g) {
      if (g == 0) {
        sched_fence();
        if constexpr (NSY == 1) {
          if (more) issue_ym(j + 1, 0);
        }
        if constexpr (DS_OUT) ds_stage();
      }
      if constexpr (DS_OUT) {
        if (g == 1) ds_fetch();
        if (g == (G > 2 ? 2 : 1)) ds_store();
      }
    };
    h8 ef[RT][NT][2];
    const auto pack_e = [&](int g) {
      ride_along(g);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) pack_group<NT>(ef[rt], tacc[rt], g);
    };
    if constexpr (kNumbered) pv_gemm_steps_numbered<RT, NT, DT, NCZ, PF, 0>(ef, zaddr, zoff, pack_e, [](int) {});
    else pv_gemm_steps<RT, NT, DT, NCZ, PF, WPE == 1>(acc, ef, zaddr, zoff, pack_e);
    if constexpr (COL) {
#pragma unroll
      for (int i = 0; i < NT * 4; ++i) rv[i] = rv_next[i];
    }
  };
  constexpr int kPeriod = NSY * NSZ / cgcd(NSY, NSZ);
  for (int j = j_begin; j < j_end; j += kPeriod) {
    static_for<kPeriod>([&](auto k_tag) {
      constexpr int k = decltype(k_tag)::value;
      if (k == 0 || j + k < j_end)
        y_tile(j + k, std::integral_constant<int, k % NSY>{}, std::integral_constant<int, k % NSZ>{});
    });
  }

  if constexpr (kNumbered) acc_settle();
  wait_vmcnt<0>();
  block_sync();
  // the staging rows are DZB wide; the global rows are DZ wide
  {
    char* const ostage = smem + wave * WM * T::kOStride;
    half_t* og = out + ((size_t)bh * seq_x + x0 + wave * WM) * DZ + dz0;
    constexpr int kChunksPerRow = DZB / 8;
    static_for<RT * DT>([&](auto i_tag) {
      constexpr int rt = decltype(i_tag)::value / DT, dt = decltype(i_tag)::value % DT;
      f16v blk;
      if constexpr (kNumbered) blk = acc_read16<16 * (rt * DT + dt)>();
      else blk = acc[rt][dt];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const h2 a = pack_rne(blk[4 * g], blk[4 * g + 1]);
        const h2 b = pack_rne(blk[4 * g + 2], blk[4 * g + 3]);
        h4 w;
        w[0] = a[0]; w[1] = a[1]; w[2] = b[0]; w[3] = b[1];
        *reinterpret_cast<h4*>(ostage + (rt * 32 + n) * T::kOStride + (32 * dt + 8 * g + 4 * h) * 2) = w;
      }
    });
    wait_lgkm0();
    constexpr int kChunks = WM * kChunksPerRow;
#pragma unroll
    for (int t = 0; t < kChunks / 64; ++t) {
      const int idx = t * 64 + lane;
      const int row = idx / kChunksPerRow, c = idx % kChunksPerRow;
      const u4v val = *reinterpret_cast<const u4v*>(ostage + row * T::kOStride + c * 16);
      *reinterpret_cast<u4v*>(reinterpret_cast<char*>(og) + (size_t)row * DZ * 2 + c * 16) = val;
    }
  }
}

}  // namespace aat
