// Wave-level tile operations shared by the forward kernels (attention and RetNet): operand fetch in
// MFMA layouts, the two contractions S^T = K Q^T and O^T += V^T P^T, and the output epilogue.
// Counterpart of reference csrc/kernels/utils/matmul.h:10-267 (smem->register + MMA pipelines), built on the
// gfx950 layouts described in cdna4.h.
#pragma once
#include "cdna4.h"

namespace aat {

// Q rows of this wave as MFMA B operands, straight from global memory.
// qrow points at element [first row of the wave + n][8*h] of a row-major [*, Kd] matrix.
// group_rows: rows from one 32-row group of the wave to the next (32: the wave's rows are contiguous).
template <int RT, int KS, int Kd>
AAT_DEV void load_q_frags(h8 (&qf)[RT][KS], const half_t* qrow, int group_rows = 32) {
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[rt][ks] = *reinterpret_cast<const h8*>(qrow + (size_t)rt * group_rows * Kd + 16 * ks);
}

// The same loads issued behind the compiler's back, into registers that already hold fragments: for a
// prefetch that stays in flight across a loop the compiler would otherwise answer with vmcnt(0) in front of
// every use of qf, LDS-DMA copies in flight included.  The caller waits (vmcnt) before the next use.
template <int RT, int KS, int Kd>
AAT_DEV void load_q_frags_async(h8 (&qf)[RT][KS], const half_t* qrow) {
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const half_t* row = qrow + (size_t)rt * 32 * Kd;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "+v"(qf[rt][ks]) : "v"(row), "n"(32 * ks) : "memory");
  }
}

// Byte offsets, inside a Rows16-swizzled [rows][Kd] tile, of this lane's A-operand chunks for tile row n.
template <int KS, int NCK, Swz MODE = Swz::Rows16>
AAT_DEV void k_frag_offsets(int (&koff)[KS], int n, int h) {
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) koff[ks] = lds_chunk_off<NCK, MODE>(n, 2 * ks + h);
}

// Byte offsets, inside a Rows4-swizzled [rows][D] tile, of the address this lane presents to the
// transposing read for d-tile dt (kv rows 4h .. 4h+3 of a 16-row step; add 8 rows for the second half).
template <int DT, int NCV, Swz MODE = Swz::Rows4>
AAT_DEV void v_frag_offsets(int (&voff)[DT], int lane) {
  const int h = lane >> 5, s16 = lane & 15;
  const int row = 4 * h + (s16 >> 2);
  const int vcol = 16 * ((lane >> 4) & 1) + 4 * (s16 & 3);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    voff[dt] = lds_chunk_off<NCV, MODE>(row, 4 * dt + (vcol >> 3)) + (vcol & 7) * 2;
}

// ---------------------------------------------------------------------------------------------------
// Explicitly scheduled contractions.  The compiler's own ordering of ds_read / MFMA / VALU leaves the
// first MFMA chain waiting on every LDS read and clusters vector work away from the matrix work, so
// the two contractions below are written as a sequence of steps -- prefetch the operand PF steps
// ahead, one MFMA group, a slice of caller-supplied vector work -- with a scheduling barrier after
// each step that pins that order.

// LDS byte address (32-bit) of a generic pointer into the dynamic LDS segment, made opaque so the
// compiler keeps the sum base+offset in a register instead of re-adding the segment base at every use.
AAT_DEV uint32_t lds_addr(const char* p) {
  uint32_t a = (uint32_t)(uintptr_t)(AAT_AS3 const char*)p;
  asm volatile("" : "+v"(a));
  return a;
}
AAT_DEV h8 lds_read_h8_at(uint32_t addr) { return *reinterpret_cast<AAT_AS3 const h8*>((uintptr_t)addr); }
AAT_DEV h4 lds_read_tr_h4_at(uint32_t addr) {
  fp16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((AAT_AS3 fp16x4_t*)(uintptr_t)addr);
  h4 o;
  __builtin_memcpy(&o, &r, 8);
  return o;
}
#ifdef AAT_NOFENCE
AAT_DEV void sched_fence() {}
#else
AAT_DEV void sched_fence() { __builtin_amdgcn_sched_barrier(0); }
#endif

// b128 LDS read issued behind the compiler's back, with the wait spelled out by the caller.  While an
// LDS-DMA copy is in flight the compiler answers every dependency on a tracked LDS load with
// lgkmcnt(0), which also waits for the prefetches issued after the fragment that is needed; LDS reads
// retire in order, so "at most N younger reads outstanding" is enough.  `imm` must fold to a constant.
AAT_DEV h8 lds_read_h8_async(uint32_t base, int imm) {
  h8 v;
  const uint32_t hi = (uint32_t)imm & ~0xffffu;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(base + hi), "i"(imm & 0xffff));
  return v;
}
// The same read at address base ^ x (x a compile-time constant): the operand addresses of a swizzled tile differ
// from one contraction step to the next by an XOR of the chunk bits, so one address register plus a one-cycle
// v_xor_b32 into a short-lived temporary serves every step where registers are scarce.
AAT_DEV h8 lds_read_h8_async_xor(uint32_t base, int x, int imm) {
  h8 v;
  uint32_t t;
  const uint32_t hi = (uint32_t)imm & ~0xffffu;
  asm volatile("v_xor_b32 %1, %3, %2\n\tds_read_b128 %0, %1 offset:%4" : "=v"(v), "=&v"(t) : "v"(base + hi), "n"(x), "i"(imm & 0xffff));
  return v;
}
// Wait until at most N LDS operations issued after the one that produced `v` are outstanding.  The
// operand ties the wait to the value, so no consumer of `v` can be scheduled above it.
template <int N> AAT_DEV void lds_wait_younger(h8& v) {
  static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit counter");
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(N));
}

// Four consecutive floats, issued the same way (per-row statistics that travel with a streamed tile).
AAT_DEV f4v lds_read_f4_async(uint32_t base, int imm) {
  f4v v;
  const uint32_t hi = (uint32_t)imm & ~0xffffu;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(base + hi), "i"(imm & 0xffff));
  return v;
}
template <int N> AAT_DEV void lds_wait_younger(f4v& a) {
  static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit counter");
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(a) : "n"(N));
}
template <int N> AAT_DEV void lds_wait_younger(f4v& a, f4v& b) {
  static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit counter");
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}

// The transposing 8-byte read (lds_read_tr_h4_at) issued the same way, and the wait for a pair of them.
AAT_DEV h4 lds_read_tr_h4_async(uint32_t base, int imm) {
  h4 v;
  const uint32_t hi = (uint32_t)imm & ~0xffffu;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(base + hi), "i"(imm & 0xffff));
  return v;
}
// Both transposing reads of one 16-row step (rows +0 and +8) at address base ^ x.
AAT_DEV void lds_read_tr_h4_pair_async_xor(h4& lo, h4& hi, uint32_t base, int x, int imm_lo, int imm_hi) {
  uint32_t t;
  asm volatile("v_xor_b32 %2, %4, %3\n\tds_read_b64_tr_b16 %0, %2 offset:%5\n\tds_read_b64_tr_b16 %1, %2 offset:%6"
               : "=v"(lo), "=&v"(hi), "=&v"(t) : "v"(base), "n"(x), "i"(imm_lo), "i"(imm_hi));
}
template <int N> AAT_DEV void lds_wait_younger(h4& a, h4& b) {
  static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit counter");
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}

// One operand read of the second contraction and its wait, either way: BLIND as above, otherwise left to the compiler.
template <bool BLIND> AAT_DEV h4 lds_read_tr_h4_either(uint32_t base, int imm) {
  if constexpr (BLIND) return lds_read_tr_h4_async(base, imm);
  else return lds_read_tr_h4_at(base + imm);
}
template <bool BLIND, int N> AAT_DEV void lds_wait_younger_either(h4& a, h4& b) {
  if constexpr (BLIND) lds_wait_younger<N>(a, b);
}

// MFMA with its accumulator forced into vector registers.  A kernel that owns more than 256 registers
// gets every compiler-issued MFMA in the form that accumulates in the 256 accumulation registers; when
// the output accumulators fill those, the short-lived score tile has to live in vector registers, which
// only a hand-written instruction can ask for.  The compiler does not see an MFMA here and inserts no
// wait states after it: mfma_settle() must stand between the last of these and any other reader.
AAT_DEV void mfma_32x32x16_vacc_first(f16v& c, h8 a, h8 b) {
  asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
}
AAT_DEV void mfma_32x32x16_vacc(f16v& c, h8 a, h8 b) {
  asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
// 24 wait states: more than the 16 passes + 3 the longest matrix instruction needs before another unit
// may read its result.
AAT_DEV void mfma_settle(f16v& c) { asm volatile("s_nop 15\n\ts_nop 7" : "+v"(c)); }

// S^T = K Q^T over one kv tile.  kaddr[ks] = LDS address of this lane's chunk for k-step ks in score
// tile 0 of the K buffer (tile nt adds nt*32 rows).  side(step) runs after the MFMA group of each step.
// VACC: accumulate in vector registers through hand-written MFMAs (see mfma_32x32x16_vacc).
// XA: only kaddr[0] is used; step ks reads at kaddr[0] ^ (ks % 8) << 5 (the Rows16 swizzle XORs the chunk index
// 2 ks + h with row bits, so the steps' addresses differ by exactly that).
// GATE0: the MFMAs of row group 0 are issued only when `group0_on` (wave-uniform) is set -- a causal wave whose early
// group no longer sees the unit while its late group does.  One code path with a branch around single instructions
// rather than a second instantiation for the late group alone: with two bodies the allocator no longer keeps the
// accumulator tuples in the same registers on both and reconciles them through scratch memory.
template <int RT, int NT, int KS, int NCK, int PF, bool VACC = false, bool XA = false, bool GATE0 = false, class Side>
AAT_DEV void qk_gemm_steps(f16v (&sacc)[RT][NT], const h8 (&qf)[RT][KS], const uint32_t (&kaddr)[KS],
                           int buf_off, Side&& side, bool group0_on = true) {
  static_assert(!GATE0 || (XA && RT == 2), "the gate is built into the in-place operand ring of two row groups");
  static_assert(!(XA && VACC), "xor addressing is for kernels that fit the unified register file");
  constexpr int S = NT * KS;
  constexpr int kTileStride = 32 * NCK * 16;
  // With rows of whole 16-chunk groups the swizzle only permutes chunks inside a group, so k-step ks
  // sits 256 bytes per group behind k-step ks % 8: eight address registers serve any contraction width.
  constexpr bool kFold = NCK % 16 == 0 && KS > 8;
  static_assert(!XA || NCK % 16 == 0 || NCK == 8, "xor addressing: the swizzle must act on whole bits of the chunk index");
  auto read = [&](int i) {
    const int ks = i % KS;
    if constexpr (XA) {
      const int imm = (NCK % 16 == 0 ? (ks / 8) * 256 : 0) + buf_off + (i / KS) * kTileStride;
      if (ks % 8 == 0) return lds_read_h8_async(kaddr[0], imm);
      return lds_read_h8_async_xor(kaddr[0], (ks % 8) << 5, imm);
    } else {
      return lds_read_h8_async(kFold ? kaddr[ks % 8] : kaddr[ks],
                               (kFold ? (ks / 8) * 256 : 0) + buf_off + (i / KS) * kTileStride);
    }
  };
  if constexpr (!VACC) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) sacc[rt][nt] = zero16();
  }
  h8 ring[PF];
#pragma unroll
  for (int i = 0; i < PF && i < S; ++i) ring[i] = read(i);
  sched_fence();
  static_for<S>([&](auto step_tag) {
    constexpr int step = decltype(step_tag)::value;
    if constexpr (XA) {
      // Scarce registers: the ring slot is consumed where it is and refilled behind its MFMAs (a matrix instruction
      // has read its operands long before an LDS read issued after it returns), so PF slots are all there is.
      lds_wait_younger<(step + PF - 1 < S) ? PF - 1 : S - 1 - step>(ring[step % PF]);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if (!GATE0 || rt != 0 || group0_on) sacc[rt][step / KS] = mfma_32x32x16(ring[step % PF], qf[rt][step % KS], sacc[rt][step / KS]);
      }
      if constexpr (step + PF < S) ring[step % PF] = read(step + PF);
    } else {
      // Wait on the slot itself, then take its value, then refill it: a copy of the value made before the wait (the
      // allocator is free to split a live range with a move) would read a register whose load has not landed.
      lds_wait_younger<(step + PF - 1 < S) ? PF - 1 : S - 1 - step>(ring[step % PF]);
      h8 cur = ring[step % PF];
      if constexpr (step + PF < S) ring[step % PF] = read(step + PF);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if constexpr (!VACC) sacc[rt][step / KS] = mfma_32x32x16(cur, qf[rt][step % KS], sacc[rt][step / KS]);
        else if constexpr (step % KS == 0) mfma_32x32x16_vacc_first(sacc[rt][step / KS], cur, qf[rt][step % KS]);
        else mfma_32x32x16_vacc(sacc[rt][step / KS], cur, qf[rt][step % KS]);
      }
    }
    side(step);
    sched_fence();
  });
  if constexpr (VACC) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) mfma_settle(sacc[rt][nt]);
  }
}

// O^T += V^T P^T over one kv tile.  vlo[dt] / vhi[dt] = LDS addresses this lane presents to the two
// transposing reads of d-tile dt (kv rows 4h..4h+3 and 8+4h..8+4h+3 of the first 16-row step; later steps
// add 16 rows, which no swizzle here sees).  pack(g) must fill pf[*][g/2][g%2] (the P operand of kv rows
// 16g .. 16g+15); it is called one group ahead of use, between MFMAs.
// BLIND: the V reads are issued behind the compiler's back like the K reads above.  In front of an LDS read it
// can see the compiler waits, with vmcnt(0), for every LDS-DMA copy in flight -- the next tile's, issued at the
// top of this one, which then has only the first contraction to arrive in instead of the whole tile.  With one
// wave on the SIMD nothing covers that wait (RetNet forward at d_qk 256 / d_v 512: -6 % with BLIND); with two or
// three another wave does, and the counted waits cost a little instead (attention forward, causal: +1.5 %).
// buf_off must fold to a constant.
template <int RT, int NT, int DT, int NCV, int PF, bool BLIND = false, class Pack>
AAT_DEV void pv_gemm_steps_hl(f16v (&oacc)[RT][DT], h8 (&pf)[RT][NT][2], const uint32_t (&vlo)[DT],
                              const uint32_t (&vhi)[DT], int buf_off, Pack&& pack) {
  constexpr int G = NT * 2;              // groups of 16 kv rows
  constexpr int S = G * DT;
  constexpr int kRow16 = 16 * NCV * 16;
  static_assert(!BLIND || 2 * PF < 16, "two reads per step in flight, counted by a 4-bit counter");
  h4 lo[PF], hi[PF];
#pragma unroll
  for (int i = 0; i < PF && i < S; ++i) {
    lo[i] = lds_read_tr_h4_either<BLIND>(vlo[i % DT], buf_off + (i / DT) * kRow16);
    hi[i] = lds_read_tr_h4_either<BLIND>(vhi[i % DT], buf_off + (i / DT) * kRow16);
  }
  pack(0);
  sched_fence();
  static_for<S>([&](auto step_tag) {
    constexpr int step = decltype(step_tag)::value;
    constexpr int g = step / DT, dt = step % DT;
    lds_wait_younger_either<BLIND, 2 * ((step + PF - 1 < S) ? PF - 1 : S - 1 - step)>(lo[step % PF], hi[step % PF]);   // wait, take, refill (qk_gemm_steps)
    h4 clo = lo[step % PF], chi = hi[step % PF];
    if constexpr (step + PF < S) {
      constexpr int nx = step + PF;
      lo[step % PF] = lds_read_tr_h4_either<BLIND>(vlo[nx % DT], buf_off + (nx / DT) * kRow16);
      hi[step % PF] = lds_read_tr_h4_either<BLIND>(vhi[nx % DT], buf_off + (nx / DT) * kRow16);
    }
    const h8 vf = cat_h4(clo, chi);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) oacc[rt][dt] = mfma_32x32x16(vf, pf[rt][g / 2][g % 2], oacc[rt][dt]);
    if constexpr (dt == 0 && g + 1 < G) pack(g + 1);
    sched_fence();
  });
}

// O^T += V^T P^T over one kv tile.  vaddr[dt] = LDS address this lane presents to the transposing read
// for d-tile dt, kv rows 0..3 (+4h) of the V buffer.  pack(g) must fill pf[*][g/2][g%2] (the P operand of
// kv rows 16g .. 16g+15); it is called one group ahead of use, between MFMAs.
// BLIND: as in pv_gemm_steps_hl.
// XA: only vaddr[0] is used; d-tile dt reads at vaddr[0] ^ (dt % 4) << 6 (the Rows4 swizzle XORs the chunk-group
// bits with row bits); implies hand-issued reads with counted waits.
// GATE0, group0_on: as in qk_gemm_steps.
template <int RT, int NT, int DT, int NCV, int PF, bool BLIND = false, bool XA = false, bool GATE0 = false, class Pack>
AAT_DEV void pv_gemm_steps(f16v (&oacc)[RT][DT], h8 (&pf)[RT][NT][2], const uint32_t (&vaddr)[DT], int buf_off,
                           Pack&& pack, bool group0_on = true) {
  static_assert(!GATE0 || (XA && RT == 2), "the gate is built into the in-place operand ring of two row groups");
  constexpr int G = NT * 2;              // groups of 16 kv rows
  constexpr int S = G * DT;
  constexpr int kRow16 = 16 * NCV * 16, kRow8 = 8 * NCV * 16;
  // The Rows4 swizzle of rows of whole 16-chunk groups exchanges chunks inside a group of 16 only, and a d-tile
  // is four chunks wide: d-tile dt sits 256 bytes per group behind d-tile dt % 4, so four address registers
  // serve any output width (the others are never read and cost nothing).
  constexpr bool kFold = NCV % 16 == 0 && DT > 4;
  static_assert(!(BLIND || XA) || 2 * PF < 16, "two reads per step in flight, counted by a 4-bit counter");
  static_assert(!XA || NCV % 16 == 0 || NCV == 8, "xor addressing: the swizzle must act on whole bits of the chunk index");
  constexpr bool kHand = BLIND || XA;
  h4 lo[PF], hi[PF];
  auto read = [&](int i, int slot) {
    const int dt = i % DT;
    if constexpr (XA) {
      const int imm = (NCV % 16 == 0 ? (dt / 4) * 256 : 0) + buf_off + (i / DT) * kRow16;
      if (dt % 4 == 0) {
        lo[slot] = lds_read_tr_h4_async(vaddr[0], imm);
        hi[slot] = lds_read_tr_h4_async(vaddr[0], imm + kRow8);
      } else {
        const int far = (imm + kRow8 > 0xffff) ? (imm & ~0x7fff) : 0;     // beyond the 16-bit offset field: one add
        lds_read_tr_h4_pair_async_xor(lo[slot], hi[slot], vaddr[0] + (uint32_t)far, (dt % 4) << 6, imm - far, imm - far + kRow8);
      }
    } else {
      const uint32_t a = kFold ? vaddr[dt % 4] : vaddr[dt];
      const int imm = (kFold ? (dt / 4) * 256 : 0) + buf_off + (i / DT) * kRow16;
      lo[slot] = lds_read_tr_h4_either<BLIND>(a, imm);
      hi[slot] = lds_read_tr_h4_either<BLIND>(a, imm + kRow8);
    }
  };
#pragma unroll
  for (int i = 0; i < PF && i < S; ++i) read(i, i);
  pack(0);
  sched_fence();
  static_for<S>([&](auto step_tag) {
    constexpr int step = decltype(step_tag)::value;
    constexpr int g = step / DT, dt = step % DT;
    if constexpr (XA) {                      // slots consumed in place and refilled behind their MFMAs (qk_gemm_steps)
      lds_wait_younger<2 * ((step + PF - 1 < S) ? PF - 1 : S - 1 - step)>(lo[step % PF], hi[step % PF]);
      const h8 vf = cat_h4(lo[step % PF], hi[step % PF]);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if (!GATE0 || rt != 0 || group0_on) oacc[rt][dt] = mfma_32x32x16(vf, pf[rt][g / 2][g % 2], oacc[rt][dt]);
      }
      if constexpr (step + PF < S) read(step + PF, step % PF);
    } else {
      lds_wait_younger_either<kHand, 2 * ((step + PF - 1 < S) ? PF - 1 : S - 1 - step)>(lo[step % PF], hi[step % PF]);   // wait, take, refill (qk_gemm_steps)
      h4 clo = lo[step % PF], chi = hi[step % PF];
      if constexpr (step + PF < S) read(step + PF, step % PF);
      const h8 vf = cat_h4(clo, chi);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) oacc[rt][dt] = mfma_32x32x16(vf, pf[rt][g / 2][g % 2], oacc[rt][dt]);
    }
    if constexpr (dt == 0 && g + 1 < G) pack(g + 1);
    sched_fence();
  });
}

// Epilogue: scale the wave's O^T accumulators per row, convert (fp16 with RNE, or fp32 as is),
// transpose through a wave-private LDS staging area and store rows with 16-byte coalesced writes.
// ostage: wave-private LDS, WM rows of O_STRIDE bytes.  og: global pointer to the wave's first output row.
// group_rows: rows in global memory from one 32-row group of the wave to the next (32: contiguous).
template <int RT, int DT, int D, int O_STRIDE, class OutT = half_t>
AAT_DEV void store_o_tile(const f16v (&oacc)[RT][DT], const float (&row_scale)[RT], char* ostage, OutT* og,
                          int lane, int group_rows = 32) {
  constexpr int kElem = (int)sizeof(OutT);
  constexpr int kChunksPerRow = D * kElem / 16, WM = RT * 32;
  const int n = lane & 31, h = lane >> 5;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float sc = row_scale[rt];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      // Accumulators that fill the accumulation registers come back one 16-register block at a time: left to
      // itself the compiler copies all of them into vector registers at the end of the main loop, and the kernel
      // spills for it.  The empty statements keep their order, so block dt is still where the MFMAs left it here.
      f16v blk = oacc[rt][dt];
      if constexpr (RT * DT * 16 >= 256) asm volatile("" : "+a"(blk));
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int d0 = 32 * dt + 8 * g + 4 * h;
        char* dst = ostage + (rt * 32 + n) * O_STRIDE + d0 * kElem;
        if constexpr (kElem == 2) {
          const h2 a = pack_rne(blk[4 * g] * sc, blk[4 * g + 1] * sc);
          const h2 b = pack_rne(blk[4 * g + 2] * sc, blk[4 * g + 3] * sc);
          h4 w;
          w[0] = a[0]; w[1] = a[1]; w[2] = b[0]; w[3] = b[1];
          *reinterpret_cast<h4*>(dst) = w;
        } else {
          f4v w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = blk[4 * g + e] * sc;
          *reinterpret_cast<f4v*>(dst) = w;
        }
      }
      if constexpr (RT * DT * 16 >= 256) sched_fence();
    }
  }
  wait_lgkm0();                                   // the staging region is private to this wave
  constexpr int kChunks = WM * kChunksPerRow;
#pragma unroll
  for (int t = 0; t < kChunks / 64; ++t) {
    const int idx = t * 64 + lane;
    const int row = idx / kChunksPerRow, c = idx % kChunksPerRow;
    const u4v val = *reinterpret_cast<const u4v*>(ostage + row * O_STRIDE + c * 16);
    const size_t grow = (size_t)(row / 32) * group_rows + row % 32;
    *reinterpret_cast<u4v*>(reinterpret_cast<char*>(og) + (grow * kChunksPerRow + c) * 16) = val;
  }
}

// fp32 output straight from the accumulators, no staging: a lane holds four consecutive columns of one row per
// accumulator group, so it stores 16-byte pieces (the two lanes of a row write neighbouring pieces).  Slower per tile
// than the staged, row-contiguous stores (about twice), which does not matter for the once-per-block partial output of a
// kv split, and it needs no LDS: a split block then occupies what its K/V buffers take and nothing more.
template <int RT, int DT, int D>
AAT_DEV void store_o_rows_f32(const f16v (&oacc)[RT][DT], const float (&row_scale)[RT], float* og, int lane) {
  const int n = lane & 31, h = lane >> 5;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const float sc = row_scale[rt];
    float* row = og + (size_t)(rt * 32 + n) * D + 4 * h;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      f16v blk = oacc[rt][dt];
      if constexpr (RT * DT * 16 >= 256) asm volatile("" : "+a"(blk));
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f4v w;
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = blk[4 * g + e] * sc;
        *reinterpret_cast<f4v*>(row + 32 * dt + 8 * g) = w;
      }
    }
  }
}

}  // namespace aat
