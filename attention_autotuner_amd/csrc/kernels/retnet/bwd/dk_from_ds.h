// RetNet backward, dK from a stored dS, for gfx950 (MI355X).
//
//     dK[kv][:] = sum_q dS[q][kv] Q[q][:]          dS = half(((dO V^T) / r) * M), B*H*S_q*S_kv fp16
//
// The chained-contraction passes (bwd_chain.h) evaluate dO V^T twice, once for dQ and once for dK: two thirds
// of either pass's matrix work.  When the caller grants a workspace of B*H*S_q*S_kv fp16 the row pass writes
// the dS tiles it forms anyway (its DS_OUT variant) and this kernel replaces the dK pass: it streams Q tiles
// and dS tiles and runs the second contraction only -- a third of the matrix work, no resident 512-wide
// fragment (128 registers), so two waves fit a SIMD.  The reference has neither (it accumulates dK in the
// registers of its single column-block kernel, csrc/kernels/retnet/bwd/bwd_colblock.h:556-576).
//
// dS lies in 64 x 64 blocks of 8 KB, [B*H][S_q/64][S_kv/64][64][64] (ds_block_offset): rows of a [S_q, S_kv]
// matrix are S_kv*2 bytes apart, a power of two at the usual lengths, so the tiles all blocks write (and read)
// at the same step of their walks would fall on the few memory channels that stride selects.  In blocks a tile
// is one contiguous piece.
//
// The row pass writes the tiles it walks and nothing else, so what lies outside its walk is garbage here:
// per query tile this kernel recomputes the kv range the writer covered (from the same mask mode, the same
// ranges and the writer's block and tile sizes) and takes dS as zero outside of it.
#pragma once
#include <type_traits>

#include "../../utils/cdna4.h"
#include "../../utils/mask_extents.h"
#include "../../utils/tile_ops.h"
#include "ds_layout.h"

namespace aat {

// Kd: width of q/k rows; BX: kv rows per block (32 per wave); BY: query rows per streamed tile; NS: LDS stages.
template <int Kd, int BX, int BY, int Nthreads, int NS>
struct RetBwdDk {
  static constexpr int NW = Nthreads / kWave;
  static constexpr int DT = Kd / 32, KSTEPS = BY / 16;
  static constexpr int NCZ = Kd / 8, NCS = 8, NSUB = BX / 64;
  static_assert(Nthreads % kWave == 0 && BX == 32 * NW, "one 32-row group of kv per wave");
  static_assert(BY == 64 && Kd % 64 == 0 && BX % 64 == 0, "a query tile is one row of dS blocks");
  static_assert(NS == 2 || NS == 3, "buffers");
  using ZDma = TileDma<BY, NCZ, Nthreads, Swz::Rows4>;   // Q tile
  using SDma = TileDma<BY * NSUB, NCS, Nthreads, Swz::Rows4, 2>;   // dS tile: NSUB consecutive blocks of BY query rows x 64 kv columns
  static constexpr int kZBytes = BY * Kd * 2, kSBytes = BY * BX * 2;
  static constexpr int kStageBytes = kZBytes + kSBytes;
  static constexpr int kTileInstr = ZDma::kIters + SDma::kIters;
  static constexpr int kOStride = Kd * 2 + 16;
  static constexpr int kMainBytes = NS * kStageBytes;
  static constexpr int kEpiBytes = BX * kOStride;
  static constexpr int kSmemBytes = kMainBytes > kEpiBytes ? kMainBytes : kEpiBytes;
};

// q [B*H, seq_q, Kd], ds in 64 x 64 blocks (above), dk [B*H, seq_k, Kd], all fp16.
// causal / extents: the mask mode of the walk, as in ret_bwd_chain (extents = the scan's ranges or nullptr).
// wr_rows x wr_cols: resident rows and streamed-tile width of the row pass that wrote ds (wr_rows % BY == 0).
template <int Kd, int BX, int BY, int Nthreads, int NS, int WPE = 2>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
ret_bwd_dk_from_ds(const half_t* __restrict__ q, const half_t* __restrict__ ds, half_t* __restrict__ dk, int H,
                   int seq_k, int seq_q, int causal, const int* __restrict__ extents, int wr_rows, int wr_cols) {
  using T = RetBwdDk<Kd, BX, BY, Nthreads, NS>;
  constexpr int DT = T::DT, KSTEPS = T::KSTEPS, NCZ = T::NCZ, NCS = T::NCS;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;

  const int Tx = seq_k / BX;
  const int tile = xcd_remap(blockIdx.x, gridDim.x);
  int bh = tile / Tx, xb = tile % Tx;
  if (causal || extents != nullptr) {             // longest blocks first: the first kv blocks
    const TileId t = causal_tile(blockIdx.x, gridDim.x, Tx, false);
    bh = t.bh;
    xb = t.blk;
  }
  const int x0 = xb * BX;
  const int diag = seq_k - seq_q;
  const int head = bh % H;
  int j_begin = 0, j_end = seq_q / BY;
  MaskExtents ext{};
  if (extents != nullptr) {
    ext = mask_extents_at(extents, H, seq_q, seq_k);
    int lo, hi;
    mask_col_range(ext, head, seq_q, seq_k, x0, BX, lo, hi);
    mask_tile_range(lo, hi, BY, j_end, j_begin, j_end);
  } else if (causal) {                            // q tiles that reach kv >= x0:  q >= x0 - diag
    const int first = x0 - diag;
    j_begin = first <= 0 ? 0 : first / BY;
  }
  // walked downwards from the end of the sequence, like the column passes of the chained kernel
  const auto tile_of = [&](int j) { return j_begin + j_end - 1 - j; };

  const char* zg = reinterpret_cast<const char*>(q + (size_t)bh * seq_q * Kd);
  const char* sg = reinterpret_cast<const char*>(ds + ds_block_offset(bh, 0, x0, seq_q, seq_k));
  const size_t s_pitch = (size_t)(seq_k >> 6) * 8192;    // from one row of blocks to the next
  typename T::ZDma zdma;
  typename T::SDma sdma;
  zdma.init(tid);
  sdma.init(tid);
  const int wave_base = wave * 64;
  auto issue = [&](int j, int st) {
    const int jt = tile_of(j);
    char* base = smem + st * T::kStageBytes;
    zdma.issue(zg + (size_t)jt * T::kZBytes, base, wave_base);
    sdma.issue(sg + (size_t)jt * s_pitch, base + T::kZBytes, wave_base);
  };

  // LDS addresses inside stage 0: Q^T fragments (A operand, d-tile dt) and this wave's dS columns (B operand);
  // both are transposing reads of rows 4h + (lane%16)/4 of a 16-row step, + 8 rows for the second half
  uint32_t zaddr[DT], saddr;
  {
    int zoff[DT];
    v_frag_offsets<DT, NCZ>(zoff, lane);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) zaddr[dt] = lds_addr(smem + zoff[dt]);
    const int s16 = lane & 15;
    const int row = (wave >> 1) * 64 + 4 * h + (s16 >> 2);         // block wave/2 of the tile, 64 rows each
    const int col = (wave & 1) * 32 + 16 * ((lane >> 4) & 1) + 4 * (s16 & 3);
    saddr = lds_addr(smem + T::kZBytes + lds_chunk_off<NCS, Swz::Rows4>(row, col >> 3) + (col & 7) * 2);
  }
  constexpr int kZRow16 = 16 * NCZ * 16, kZRow8 = 8 * NCZ * 16, kSRow16 = 16 * NCS * 16, kSRow8 = 8 * NCS * 16;

  f16v acc[1][DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc[0][dt] = zero16();

  if (j_begin < j_end) {
    issue(j_begin, 0);
    if constexpr (NS == 3) {
      if (j_begin + 1 < j_end) issue(j_begin + 1, 1);
    }
  }
  const int my_kv = x0 + wave * 32 + n;           // the kv position this lane owns

  auto q_tile = [&](const int j, auto st_tag) {
    constexpr int st = decltype(st_tag)::value;
    constexpr int off = st * T::kStageBytes;
    const bool more = (j + 1 < j_end);
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

    // the kv range the writer covered for the row block this query tile lies in
    const int jt = tile_of(j);
    const int wx0 = (jt * BY) / wr_rows * wr_rows;
    int wlo = 0, whi = seq_k;
    if (extents != nullptr) {
      int lo, hi, jb, je;
      mask_row_range(ext, head, seq_q, wx0, wr_rows, lo, hi);
      mask_tile_range(lo, hi, wr_cols, seq_k / wr_cols, jb, je);
      wlo = jb * wr_cols;
      whi = je * wr_cols;
    } else if (causal) {
      const int last = wx0 + wr_rows - 1 + diag;
      const int lim = last < 0 ? 0 : last / wr_cols + 1;
      whi = lim * wr_cols < seq_k ? lim * wr_cols : seq_k;
    }
    const bool all_written = wlo <= x0 && x0 + BX <= whi;          // block-uniform
    const bool mine_written = my_kv >= wlo && my_kv < whi;

    // The operand reads are issued as instructions with counted waits (tile_ops.h): in front of an LDS read it can see
    // the compiler waits for every LDS-DMA copy in flight, i.e. for the next tile this one has just requested.
    constexpr int PF = 2;
    static_for<KSTEPS>([&](auto s_tag) {
      constexpr int s = decltype(s_tag)::value;
      h4 blo = lds_read_tr_h4_async(saddr, off + s * kSRow16);
      h4 bhi = lds_read_tr_h4_async(saddr, off + s * kSRow16 + kSRow8);
      h4 lo[PF], hi[PF];
#pragma unroll
      for (int i = 0; i < PF && i < DT; ++i) {
        lo[i] = lds_read_tr_h4_async(zaddr[i], off + s * kZRow16);
        hi[i] = lds_read_tr_h4_async(zaddr[i], off + s * kZRow16 + kZRow8);
      }
      h8 bf;
      static_for<DT>([&](auto dt_tag) {
        constexpr int dt = decltype(dt_tag)::value;
        // wait on the slot, take its value, refill it (a copy made before the wait could read a register whose load
        // has not landed); the B pair is older: it has landed too
        lds_wait_younger<2 * ((dt + PF - 1 < DT) ? PF - 1 : DT - 1 - dt)>(lo[dt % PF], hi[dt % PF]);
        h4 clo = lo[dt % PF], chi = hi[dt % PF];
        if constexpr (dt + PF < DT) {
          lo[dt % PF] = lds_read_tr_h4_async(zaddr[dt + PF], off + s * kZRow16);
          hi[dt % PF] = lds_read_tr_h4_async(zaddr[dt + PF], off + s * kZRow16 + kZRow8);
        }
        if constexpr (dt == 0) {
          asm volatile("" : "+v"(blo), "+v"(bhi));
          bf = cat_h4(blo, bhi);
          if (!all_written) {
            if (!mine_written) {
#pragma unroll
              for (int e = 0; e < 8; ++e) bf[e] = (half_t)0.f;
            }
          }
        }
        acc[0][dt] = mfma_32x32x16(cat_h4(clo, chi), bf, acc[0][dt]);
      });
    });
  };
  for (int j = j_begin; j < j_end; j += NS) {
    static_for<NS>([&](auto k_tag) {
      constexpr int k = decltype(k_tag)::value;
      if (k == 0 || j + k < j_end) q_tile(j + k, std::integral_constant<int, k>{});
    });
  }

  wait_vmcnt<0>();
  block_sync();
  const float one[1] = {1.f};
  store_o_tile<1, DT, Kd, T::kOStride>(acc, one, smem + wave * 32 * T::kOStride,
                                       dk + ((size_t)bh * seq_k + x0 + wave * 32) * Kd, lane);
}

}  // namespace aat
