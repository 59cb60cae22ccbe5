// Output accumulators held in the accumulation registers by number, outside the compiler's register allocation.
//
// A kernel that runs one wave per SIMD owns 512 registers: 256 vector registers and 256 accumulation registers that only
// matrix instructions and v_accvgpr_read/write can touch.  A register-fused forward kernel with a wide value head fills
// all 256 of the latter with its output tile (32 rows x 512 columns per wave).  Handed to the compiler as ordinary values,
// such a tile is a constant struggle: any change of the loop around it (a second buffer parity, a copy threaded between
// the matrix steps, a branch) can make the allocator place the sixteen 16-register tuples differently at two points of
// the program and reconcile the two placements through scratch memory, hundreds of bytes per lane and tile.  Here the
// tile never becomes a C++ value: matrix instruction, rescale, zero and read-out name their registers a[LO:LO+15]
// literally, and one statement at the top of the kernel claims the whole file so that the compiler allocates it to the
// kernel and keeps nothing of its own there.  What the compiler then allocates is an ordinary kernel of ~150 vector
// registers.
//
// The compiler knows nothing of these registers, so the wait states it would insert are the caller's:
//   * acc_settle() between the last matrix instruction and a read-out (acc_read, acc_scale);
//   * acc_scale ends with the wait states a matrix instruction needs after v_accvgpr_write.
// Matrix instructions that accumulate into the same tuple back to back are interlocked by the hardware.
#pragma once
#include "cdna4.h"
#include "tile_ops.h"

namespace aat {

#define AAT_D10(p) p "0", p "1", p "2", p "3", p "4", p "5", p "6", p "7", p "8", p "9"
#define AAT_AGPR_ALL                                                                                                  \
  AAT_D10("a"), AAT_D10("a1"), AAT_D10("a2"), AAT_D10("a3"), AAT_D10("a4"), AAT_D10("a5"), AAT_D10("a6"),             \
      AAT_D10("a7"), AAT_D10("a8"), AAT_D10("a9"), AAT_D10("a10"), AAT_D10("a11"), AAT_D10("a12"), AAT_D10("a13"),     \
      AAT_D10("a14"), AAT_D10("a15"), AAT_D10("a16"), AAT_D10("a17"), AAT_D10("a18"), AAT_D10("a19"), AAT_D10("a20"),  \
      AAT_D10("a21"), AAT_D10("a22"), AAT_D10("a23"), AAT_D10("a24"), "a250", "a251", "a252", "a253", "a254", "a255"

// Claim all 256 accumulation registers for the kernel (call once, first thing).  The comment it leaves in the kernel's
// assembly marks the kernel for the build's check that the compiler has kept out of the file (autotuner/codegen.py:
// foreign_accumulator_use): without it the check takes the kernel for ordinary MFMA code, so every kernel that uses
// the functions below must call this.
AAT_DEV void acc_claim_all() { asm volatile("; aat: accumulation registers addressed by number" ::: AAT_AGPR_ALL); }

// a[LO : LO+15] += A x B (32x32x16, fp16 operands).
template <int LO> AAT_DEV void acc_mfma_32x32x16(const h8& a, const h8& b) {
  static_assert(LO >= 0 && LO + 16 <= 256 && LO % 16 == 0, "one 16-register tuple of the accumulation file");
  asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(a), "v"(b), "n"(LO), "n"(LO + 15));
}

// a[LO : LO+N) = 0.
template <int LO, int N> AAT_DEV void acc_zero() {
  static_for<N>([&](auto i_tag) {
    constexpr int R = LO + decltype(i_tag)::value;
    asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(R));
  });
}

// More wait states than the longest matrix instruction (16 passes + 3) needs before another unit may read its result.
AAT_DEV void acc_settle() { asm volatile("s_nop 15\n\ts_nop 7"); }

// a[LO : LO+N) *= alpha (per lane).  The caller has let the matrix instructions settle.
template <int LO, int N> AAT_DEV void acc_scale(float alpha) {
  static_for<N>([alpha](auto i_tag) {
    constexpr int R = LO + decltype(i_tag)::value;
    float t;
    asm volatile("v_accvgpr_read_b32 %0, a[%2]\n\tv_mul_f32 %0, %1, %0\n\tv_accvgpr_write_b32 a[%2], %0"
                 : "=&v"(t) : "v"(alpha), "n"(R));
  });
  asm volatile("s_nop 3");             // v_accvgpr_write -> matrix instruction reading the register as its addend
}

// One 16-register tuple read out (after acc_settle).
template <int LO> AAT_DEV f16v acc_read16() {
  f16v r;
  static_for<16>([&r](auto i_tag) {
    constexpr int I = decltype(i_tag)::value;
    float t;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t) : "n"(LO + I));
    r[I] = t;
  });
  return r;
}

// O^T += V^T P^T over one kv tile into the numbered accumulators: row group rt, d-tile dt accumulate in
// a[BASE + 16 (rt DT + dt) ...].  Operand reads hand-issued with counted waits as in pv_gemm_steps (BLIND);
// pack(g) and side(step) as there.
// buf_off must fold to a constant.
template <int RT, int NT, int DT, int NCV, int PF, int BASE, class Pack, class Side>
AAT_DEV void pv_gemm_steps_numbered(h8 (&pf)[RT][NT][2], const uint32_t (&vaddr)[DT], int buf_off, Pack&& pack, Side&& side) {
  constexpr int G = NT * 2;              // groups of 16 kv rows
  constexpr int S = G * DT;
  constexpr int kRow16 = 16 * NCV * 16, kRow8 = 8 * NCV * 16;
  constexpr bool kFold = NCV % 16 == 0 && DT > 4;      // as in pv_gemm_steps: four address registers serve any width
  static_assert(2 * PF < 16, "two reads per step in flight, counted by a 4-bit counter");
  static_assert(BASE + RT * DT * 16 <= 256, "the accumulation file has 256 registers");
  h4 lo[PF], hi[PF];
  auto read = [&](int i, int slot) {
    const int dt = i % DT;
    const uint32_t a = kFold ? vaddr[dt % 4] : vaddr[dt];
    const int imm = (kFold ? (dt / 4) * 256 : 0) + buf_off + (i / DT) * kRow16;
    lo[slot] = lds_read_tr_h4_async(a, imm);
    hi[slot] = lds_read_tr_h4_async(a, imm + kRow8);
  };
#pragma unroll
  for (int i = 0; i < PF && i < S; ++i) read(i, i);
  pack(0);
  asm volatile("s_nop 1");               // packed by vector instructions, read by a matrix instruction the compiler does not see
  sched_fence();
  static_for<S>([&](auto step_tag) {
    constexpr int step = decltype(step_tag)::value;
    constexpr int g = step / DT, dt = step % DT;
    lds_wait_younger<2 * ((step + PF - 1 < S) ? PF - 1 : S - 1 - step)>(lo[step % PF], hi[step % PF]);   // wait, take, refill (qk_gemm_steps)
    h4 clo = lo[step % PF], chi = hi[step % PF];
    if constexpr (step + PF < S) read(step + PF, step % PF);
    const h8 vf = cat_h4(clo, chi);
    static_for<RT>([&](auto rt_tag) {
      constexpr int rt = decltype(rt_tag)::value;
      acc_mfma_32x32x16<BASE + 16 * (rt * DT + dt)>(vf, pf[rt][g / 2][g % 2]);
    });
    if constexpr (dt == 0 && g + 1 < G) {
      pack(g + 1);
      asm volatile("s_nop 1");
    }
    side(step);
    sched_fence();
  });
}

// store_o_tile for numbered accumulators (after acc_settle): scale per row, round to fp16, transpose through the
// wave-private staging area, store rows with 16-byte writes.
template <int RT, int DT, int D, int O_STRIDE, int BASE>
AAT_DEV void store_o_tile_numbered(const float (&row_scale)[RT], char* ostage, half_t* og, int lane) {
  constexpr int kChunksPerRow = D * 2 / 16, WM = RT * 32;
  const int n = lane & 31, h = lane >> 5;
  static_for<RT * DT>([&](auto i_tag) {
    constexpr int rt = decltype(i_tag)::value / DT, dt = decltype(i_tag)::value % DT;
    const float sc = row_scale[rt];
    const f16v blk = acc_read16<BASE + 16 * (rt * DT + dt)>();
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const h2 a = pack_rne(blk[4 * g] * sc, blk[4 * g + 1] * sc);
      const h2 b = pack_rne(blk[4 * g + 2] * sc, blk[4 * g + 3] * sc);
      h4 w;
      w[0] = a[0]; w[1] = a[1]; w[2] = b[0]; w[3] = b[1];
      *reinterpret_cast<h4*>(ostage + (rt * 32 + n) * O_STRIDE + (32 * dt + 8 * g + 4 * h) * 2) = w;
    }
    sched_fence();
  });
  wait_lgkm0();                                   // the staging region is private to this wave
  constexpr int kChunks = WM * kChunksPerRow;
#pragma unroll
  for (int t = 0; t < kChunks / 64; ++t) {
    const int idx = t * 64 + lane;
    const int row = idx / kChunksPerRow, c = idx % kChunksPerRow;
    const u4v val = *reinterpret_cast<const u4v*>(ostage + row * O_STRIDE + c * 16);
    *reinterpret_cast<u4v*>(reinterpret_cast<char*>(og) + ((size_t)row * kChunksPerRow + c) * 16) = val;
  }
}

}  // namespace aat
