// Building blocks of the LDS-fused ("smemfuse") forward kernels.
//
// In the register-fused kernels every wave owns whole query rows for both contractions.  Here the
// two contractions use different wave grids (reference: the warps_mma1_N / warps_mma_N parameters of
// csrc/kernels/attention/smemfuse/smemfuse.h:61-62 and :343-452): for S^T = K Q^T the NW waves form a
// W1M x W1N grid over (query rows, kv columns); P is rounded to fp16 and parked in LDS; for
// O^T += V^T P^T the waves form a W2M x W2N grid over (query rows, d columns) and read P back in MFMA
// B-operand order.  A wave's output accumulator then covers Br*D/NW elements whatever the row count,
// so a small Br keeps a wide D (e.g. 512) inside the register file, and each V element is read from
// LDS by W2M waves instead of by all of them.
//
// Unlike the reference, scores never visit LDS in fp32: each wave keeps its S^T sub-tile in registers
// and only the per-row partial statistics (max / sum / abs-sum) are exchanged through LDS.
#pragma once
#include "cdna4.h"
#include "tile_ops.h"

namespace aat {

template <int Br, int Bc, int D, int Nthreads, int W1N, int W2N>
struct SmemFuseGrid {
  static constexpr int NW = Nthreads / kWave;
  static_assert(NW % W1N == 0 && NW % W2N == 0, "wave grids must tile the block");
  static constexpr int W1M = NW / W1N, W2M = NW / W2N;
  static constexpr int RM1 = Br / W1M, CN1 = Bc / W1N;      // rows x kv columns per wave, first contraction
  static constexpr int RM2 = Br / W2M, DN2 = D / W2N;       // rows x d columns per wave, second contraction
  static_assert(Br % W1M == 0 && RM1 % 32 == 0 && Bc % W1N == 0 && CN1 % 32 == 0, "first wave grid");
  static_assert(Br % W2M == 0 && RM2 % 32 == 0 && D % W2N == 0 && DN2 % 32 == 0, "second wave grid");
  static constexpr int RT1 = RM1 / 32, NT1 = CN1 / 32, RT2 = RM2 / 32, DT2 = DN2 / 32;
  static constexpr int kPStride = Bc * 2 + 16;              // bytes per P row in LDS (padded: conflict-free b128 reads)
  static constexpr int kPBytes = Br * kPStride;
  // per-row exchange area: W1N partial statistics, one rescale factor, one flag word per wave
  static constexpr int kStatBytes = (W1N * Br + Br) * 4 + 64;
  static constexpr int kOStride = DN2 * 2 + 16;             // epilogue staging row stride
  static constexpr int kEpiBytes = NW * RM2 * kOStride;
};

// Park a wave's P sub-tile (fp32 in the S^T accumulator layout) in LDS as fp16, row-major [q][kv].
// prow = LDS address of (this lane's query row of row group 0, this wave's first kv column) + 8*h bytes.
template <int RT, int NT, int P_STRIDE>
AAT_DEV void store_p(const f16v (&s)[RT][NT], uint32_t prow) {
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const h2 a = pack_rne(s[rt][nt][4 * g], s[rt][nt][4 * g + 1]);
        const h2 b = pack_rne(s[rt][nt][4 * g + 2], s[rt][nt][4 * g + 3]);
        h4 w;
        w[0] = a[0]; w[1] = a[1]; w[2] = b[0]; w[3] = b[1];
        *reinterpret_cast<AAT_AS3 h4*>((uintptr_t)(prow + rt * 32 * P_STRIDE + (32 * nt + 8 * g) * 2)) = w;
      }
}

// O^T += V^T P^T with P read back from LDS.  k-step s covers kv rows 16s .. 16s+15; lane half h
// contracts rows 16s + 8h .. +7 (8 contiguous fp16 of its P row; two transposed 4-row reads of V).
// paddr[rt] = LDS address of this lane's P row of row group rt, + 16*h bytes.
// vaddr[dt] = address presented to the transposing read for d-tile dt, kv rows 8h + (lane%16)/4.
template <int RT, int DT, int KSTEPS, int NCV>
AAT_DEV void pv_gemm_from_lds(f16v (&oacc)[RT][DT], const uint32_t (&paddr)[RT], const uint32_t (&vaddr)[DT],
                              int vbuf_off) {
  constexpr int kRow16 = 16 * NCV * 16, kRow4 = 4 * NCV * 16;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    h8 pfrag[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) pfrag[rt] = lds_read_h8_at(paddr[rt] + s * 32);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const h4 lo = lds_read_tr_h4_at(vaddr[dt] + vbuf_off + s * kRow16);
      const h4 hi = lds_read_tr_h4_at(vaddr[dt] + vbuf_off + s * kRow16 + kRow4);
      const h8 vf = cat_h4(lo, hi);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) oacc[rt][dt] = mfma_32x32x16(vf, pfrag[rt], oacc[rt][dt]);
    }
  }
}

// Addresses for pv_gemm_from_lds: V^T operand of d-tile (d_tile0 + dt), rows 8h + (lane%16)/4 of a 16-row step.
template <int DT, int NCV>
AAT_DEV void v_frag_addrs_8(uint32_t (&vaddr)[DT], const char* vbuf, int lane, int d_tile0) {
  const int h = lane >> 5, s16 = lane & 15;
  const int row = 8 * h + (s16 >> 2);
  const int vcol = 16 * ((lane >> 4) & 1) + 4 * (s16 & 3);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    vaddr[dt] = lds_addr(vbuf + lds_chunk_off<NCV, Swz::Rows4>(row, 4 * (d_tile0 + dt) + (vcol >> 3)) + (vcol & 7) * 2);
}

// Epilogue for a (rows x d-slice) accumulator: scale per row, round, transpose through wave-private LDS,
// store with 16-byte writes.  og points at global element [first row of the wave][first d of the slice].
template <int RT, int DT, int D, int O_STRIDE>
AAT_DEV void store_o_slice(const f16v (&oacc)[RT][DT], const float (&row_scale)[RT], char* ostage, half_t* og, int lane) {
  constexpr int kChunksPerRow = DT * 4, WM = RT * 32;
  const int n = lane & 31, h = lane >> 5;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float sc = row_scale[rt];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const h2 a = pack_rne(oacc[rt][dt][4 * g] * sc, oacc[rt][dt][4 * g + 1] * sc);
        const h2 b = pack_rne(oacc[rt][dt][4 * g + 2] * sc, oacc[rt][dt][4 * g + 3] * sc);
        h4 w;
        w[0] = a[0]; w[1] = a[1]; w[2] = b[0]; w[3] = b[1];
        *reinterpret_cast<h4*>(ostage + (rt * 32 + n) * O_STRIDE + (32 * dt + 8 * g + 4 * h) * 2) = w;
      }
  }
  wait_lgkm0();
  constexpr int kChunks = WM * kChunksPerRow;
#pragma unroll
  for (int t = 0; t < (kChunks + 63) / 64; ++t) {
    const int idx = t * 64 + lane;
    if (idx < kChunks) {
      const int row = idx / kChunksPerRow, c = idx % kChunksPerRow;
      const u4v val = *reinterpret_cast<const u4v*>(ostage + row * O_STRIDE + c * 16);
      *reinterpret_cast<u4v*>(reinterpret_cast<char*>(og) + (size_t)row * D * 2 + c * 16) = val;
    }
  }
}

}  // namespace aat
