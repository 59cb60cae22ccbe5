// CDNA4 (gfx950) primitives shared by every kernel template in this tree: vector types, the
// 32x32x16 fp16 MFMA, LDS-DMA tile copies, swizzled LDS addressing, barriers with explicit wait
// counts, RNE fp16 packing and the lane<->lane^32 exchange used by all row reductions.
//
// This file plays the part that csrc/kernels/utils/{gmem_copy,matmul,misc}.h play in the reference
// (reference: csrc/kernels/utils/gmem_copy.h:41-202, matmul.h:10-267, misc.h:7-67), but nothing here is
// derived from CuTe: the layouts below are the native MFMA operand layouts of a 64-lane wavefront.
//
// MFMA v_mfma_f32_32x32x16_f16, one wave, lane l, half h = l/32, column n = l%32:
//   A (32 x 16): lane holds A[n][8h .. 8h+7]          (8 halfs, one 16-byte chunk)
//   B (16 x 32): lane holds B[8h .. 8h+7][n]
//   C (32 x 32): lane holds C[8*(v/4) + 4h + v%4][n]  for v = 0..15
// The contraction pairs slot (h, j) of A with slot (h, j) of B, so any consistent assignment of real
// k indices to slots is valid.  All kernels here compute the *transposed* score tile S^T = K * Q^T:
// then a lane owns ONE query row (n) and 16 of every 32 kv positions, row reductions are in-lane plus
// one exchange with lane^32, and the C registers of S^T are already a valid B operand for O^T = V^T * P^T.
#pragma once
#include <type_traits>
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace aat {

typedef _Float16 half_t;
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef __fp16 fp16x4_t __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f2v __attribute__((ext_vector_type(2)));
typedef unsigned int u2v __attribute__((ext_vector_type(2)));
typedef unsigned int u4v __attribute__((ext_vector_type(4)));

#define AAT_DEV __device__ __forceinline__
#define AAT_AS1 __attribute__((address_space(1)))
#define AAT_AS3 __attribute__((address_space(3)))

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// ---------------------------------------------------------------------------------------------------
// MFMA
AAT_DEV f16v mfma_32x32x16(h8 a, h8 b, f16v c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
AAT_DEV f16v zero16() {
  f16v z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}
// Row of the 32x32 C tile that accumulator register v of a lane in half h holds.
AAT_DEV constexpr int c_row(int v, int h) { return 8 * (v >> 2) + 4 * h + (v & 3); }

// ---------------------------------------------------------------------------------------------------
// Wait counters and barriers.  s_barrier is issued through inline asm with a memory clobber so the
// compiler keeps LDS accesses on their side of it; the hardware waits are spelled out by the caller
// (vmcnt covers global loads AND LDS-DMA writes, lgkmcnt covers ds_read/ds_write).
template <int N> AAT_DEV void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
AAT_DEV void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// vmcnt(0) as an instruction the compiler can see.  Its own bookkeeping of outstanding loads does not read the waits
// written in asm: fragments loaded ahead of a loop stay "possibly in flight" at the loop header for good, and it guards
// their first use in the loop body with counted vmcnt waits on every iteration -- which, in hardware, also wait for the
// LDS-DMA copies of the next tile issued a moment earlier (vmcnt(0) by the last fragment: no overlap left).  One visible
// wait between those loads and the loop settles the books.
AAT_DEV void wait_vmcnt0_visible() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0), expcnt and lgkmcnt untouched
// Workgroup barrier that makes this thread's finished LDS traffic (ds ops and, when the caller has
// already waited on vmcnt, LDS-DMA writes) visible to the other waves of the block.
AAT_DEV void block_sync() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---------------------------------------------------------------------------------------------------
// Swizzles over 16-byte chunk indices of a row-major fp16 tile in LDS.  NC = chunks per row
// (a multiple of 8 because every head dimension is a multiple of 64).  LDS has 64 banks x 4 B; a
// ds_read_b128 is served 16 lanes per cycle, a ds_read_b64 32 lanes per cycle.
//
// swz_rows16: for "16 consecutive rows, same chunk" reads (MFMA A/B operand fetched as one b128 per
// lane, rows across lanes).  Conflict-free for NC in {8,16,32,64}; 2-way for the other multiples of 8.
template <int NC> AAT_DEV constexpr int swz_rows16(int row, int c) {
  if constexpr (NC % 16 == 0) return c ^ (row & 15);
  else if constexpr (NC == 8) return c ^ ((row >> 1) & 7);
  else if constexpr (NC == 4) return c ^ ((row >> 2) & 3);
  else return c ^ (row & 7);
}
// swz_rows4: for the transposing read ds_read_b64_tr_b16, where one 32-lane phase touches 4
// consecutive rows x 64 contiguous bytes.  Conflict-free for every NC that is a multiple of 8.
template <int NC> AAT_DEV constexpr int swz_rows4(int row, int c) {
  if constexpr (NC % 16 == 0) return c ^ ((row & 3) << 2);
  else return c ^ (((row >> 1) & 1) << 2);
}

// ---------------------------------------------------------------------------------------------------
// LDS-DMA tile copy (global_load_lds_dwordx4): each lane names a 16-byte global source, the hardware
// writes lane i's data at  lds_base + 16*i  with lds_base wave-uniform.  No VGPR staging; completion is
// tracked by vmcnt.  A tile of ROWS x (NC*8) halfs is ROWS*NC chunks; thread t of NT copies chunks
// t, t+NT, ...  Chunk slot s sits at LDS byte 16*s and holds global chunk (row = s/NC, c = SWZ(row, s%NC)).
enum class Swz { Rows16, Rows4, Both };

// swz_both: one tile read BOTH ways (b128 operand reads of 16 consecutive rows and transposing reads of
// 4 consecutive rows x 4 chunks).  The XOR term must be a bijection of the row bits that a b128 phase
// walks (so 16 rows of one chunk hit 16 different slots) whose chunk-group bits also change with the two
// low row bits (so the 4 rows of a transposing phase hit 4 different 64-byte groups).
template <int NC> AAT_DEV constexpr int swz_both(int row, int c) {
  if constexpr (NC % 16 == 0) {
    return c ^ ((row & 15) ^ ((row & 3) << 2));                      // (b3^b1, b2^b0, b1, b0)
  } else {
    // an odd number of 128-byte halves per row (64, 192, 320 ... halfs): consecutive rows start on alternating halves
    // of a 256-byte line, so the row's lowest bit already separates them and the XOR term, which stays inside a group
    // of 8 chunks, is a bijection of the other three
    static_assert(NC % 16 == 8, "tiles read both ways are a multiple of 64 halfs wide");
    const int b1 = (row >> 1) & 1, b2 = (row >> 2) & 1, b3 = (row >> 3) & 1;
    return c ^ (((b3 ^ b1) << 2) | (b2 << 1) | b1);
  }
}

template <int NC, Swz MODE> AAT_DEV constexpr int swz(int row, int c) {
  if constexpr (MODE == Swz::Rows16) return swz_rows16<NC>(row, c);
  else if constexpr (MODE == Swz::Rows4) return swz_rows4<NC>(row, c);
  else return swz_both<NC>(row, c);
}

// Compile-time proof that the swizzles do what they are for.  LDS serves 256 bytes per cycle: the 16
// lanes of a b128 phase (16 consecutive rows, one logical chunk) and the 32 lanes of a transposing b64
// phase (4 consecutive rows x 4 consecutive chunks) must each touch 16 different 16-byte slots mod 256.
template <int NC, Swz MODE> constexpr bool b128_phase_conflict_free() {
  for (int r0 = 0; r0 < 32; r0 += 16)
    for (int c = 0; c < NC; ++c) {
      unsigned seen = 0;
      for (int i = 0; i < 16; ++i) {
        const unsigned slot = ((r0 + i) * NC + swz<NC, MODE>(r0 + i, c)) % 16;
        if (seen >> slot & 1u) return false;
        seen |= 1u << slot;
      }
    }
  return true;
}
template <int NC, Swz MODE> constexpr bool transposing_phase_conflict_free() {
  for (int r0 = 0; r0 < 32; r0 += 4)
    for (int g = 0; g < NC / 4; ++g) {
      unsigned seen = 0;
      for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j) {
          const unsigned slot = ((r0 + i) * NC + swz<NC, MODE>(r0 + i, 4 * g + j)) % 16;
          if (seen >> slot & 1u) return false;
          seen |= 1u << slot;
        }
    }
  return true;
}
static_assert(b128_phase_conflict_free<8, Swz::Rows16>() && b128_phase_conflict_free<16, Swz::Rows16>() &&
              b128_phase_conflict_free<32, Swz::Rows16>() && b128_phase_conflict_free<64, Swz::Rows16>(),
              "operand reads of 64/128/256/512-wide tiles are conflict-free");
static_assert(transposing_phase_conflict_free<8, Swz::Rows4>() && transposing_phase_conflict_free<16, Swz::Rows4>() &&
              transposing_phase_conflict_free<24, Swz::Rows4>() && transposing_phase_conflict_free<32, Swz::Rows4>() &&
              transposing_phase_conflict_free<64, Swz::Rows4>(),
              "transposing reads of 64..512-wide tiles are conflict-free");
static_assert(b128_phase_conflict_free<8, Swz::Both>() && transposing_phase_conflict_free<8, Swz::Both>() &&
              b128_phase_conflict_free<16, Swz::Both>() && transposing_phase_conflict_free<16, Swz::Both>() &&
              b128_phase_conflict_free<24, Swz::Both>() && transposing_phase_conflict_free<24, Swz::Both>() &&
              b128_phase_conflict_free<32, Swz::Both>() && transposing_phase_conflict_free<32, Swz::Both>() &&
              b128_phase_conflict_free<40, Swz::Both>() && transposing_phase_conflict_free<40, Swz::Both>() &&
              b128_phase_conflict_free<48, Swz::Both>() && transposing_phase_conflict_free<48, Swz::Both>() &&
              b128_phase_conflict_free<56, Swz::Both>() && transposing_phase_conflict_free<56, Swz::Both>() &&
              b128_phase_conflict_free<64, Swz::Both>() && transposing_phase_conflict_free<64, Swz::Both>(),
              "tiles read both ways (every multiple of 64 halfs up to 512) are conflict-free for both access patterns");

constexpr int cgcd(int a, int b) { return b == 0 ? a : cgcd(b, a % b); }

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), in order.
template <int N, int I = 0, class F> AAT_DEV void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

// The source address of every copy is split into a wave-uniform part (tile pointer + a compile-time
// multiple of the row pitch, kept in SGPRs) and one 32-bit per-lane offset, so a tile copy costs one
// or two VGPRs of addressing instead of a 64-bit pointer per instruction.  That works when the block's
// threads cover whole rows per instruction (NT % NC == 0): then a thread keeps its chunk column and
// only the swizzle term can change from one instruction to the next, with a short period.
// AUX: cache-policy bits of the load (2 = non-temporal: data read once).
// SADDR: the copy instruction is written out in its scalar-base form (64-bit base in SGPRs, one 32-bit per-lane
// offset) with its own write of M0; the builtin form adds the per-lane offset to the base as a 64-bit vector add per
// instruction and keeps the offsets as register pairs.  A kernel must issue all its copies one way or the other: the
// compiler does not know that the asm form has changed M0.
template <int ROWS, int NC, int NT, Swz MODE, int AUX = 0, bool SADDR = false>
struct TileDma {
  static constexpr int kChunks = ROWS * NC;
  static_assert(kChunks % NT == 0, "tile chunks must divide evenly over the block's threads");
  static constexpr int kIters = kChunks / NT;          // LDS-DMA instructions per thread per tile
  static constexpr int kBytes = kChunks * 16;
  static constexpr int kRowBytes = NC * 16;
  static constexpr bool kRegular = (NT % NC == 0);
  static constexpr int kRowsPerIter = kRegular ? NT / NC : 1;
  static constexpr int kPeriod = (MODE == Swz::Rows4) ? 4 : 16;    // rows after which the swizzle repeats
  static constexpr int kDistinctRaw = kPeriod / cgcd(kRowsPerIter, kPeriod);
  static constexpr int kDistinct = !kRegular ? kIters : (kDistinctRaw < kIters ? kDistinctRaw : kIters);
  uint32_t loff[kDistinct];                            // per-lane byte offsets inside a tile

  int pitch;                                           // bytes between consecutive tile rows in global memory

  // `row_pitch_bytes`: distance between rows of the source matrix (defaults to a dense tile-wide matrix).
  AAT_DEV void init(int tid, int row_pitch_bytes = kRowBytes) {
    pitch = row_pitch_bytes;
#pragma unroll
    for (int i = 0; i < kDistinct; ++i) {
      const int s = i * NT + tid;
      const int row = s / NC, cs = s % NC;
      const int row0 = kRegular ? tid / NC : row;      // the uniform part carries i * kRowsPerIter rows
      loff[i] = (uint32_t)(row0 * pitch + swz<NC, MODE>(row, cs) * 16);
    }
  }
  // Issue the copy of one tile.  `g` points at the tile's first row in global memory (wave-uniform),
  // `lds` at the destination buffer (block-uniform); wave_base = 64 * wave index (wave-uniform).
  AAT_DEV void issue(const char* g, char* lds, int wave_base) const { issue_part<0, kIters>(g, lds, wave_base); }

  // Instructions [I0, I1) only.  With kRegular, instruction i covers tile rows
  // [i*kRowsPerIter, (i+1)*kRowsPerIter), so this copies a contiguous range of rows.
  template <int I0, int I1>
  AAT_DEV void issue_part(const char* g, char* lds, int wave_base) const {
#pragma unroll
    for (int i = I0; i < I1; ++i) issue_one(i, g, lds, wave_base);
  }
  // Instruction i alone (i must fold to a constant where this is inlined): lets a caller thread the
  // copy of a tile between other instructions one LDS-DMA instruction at a time.
  AAT_DEV void issue_one(int i, const char* g, char* lds, int wave_base) const {
    uint64_t base = (uint64_t)(uintptr_t)(kRegular ? g + (size_t)i * kRowsPerIter * pitch : g);
    asm volatile("" : "+s"(base));                     // keep the uniform part in SGPRs (saddr form)
    const uint32_t lane_off = loff[kRegular ? i % kDistinct : i];
    if constexpr (SADDR) {
      static_assert(AUX == 0 || !SADDR, "the scalar-base form is written without cache-policy bits");
      const uint32_t dst = __builtin_amdgcn_readfirstlane(
          (uint32_t)(uintptr_t)(AAT_AS3 char*)(lds + (i * NT + wave_base) * 16));
      asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(lane_off), "s"(base) : "memory");
      return;
    }
    __builtin_amdgcn_global_load_lds((const AAT_AS1 void*)(uintptr_t)(base + lane_off),
                                     (AAT_AS3 void*)(lds + (i * NT + wave_base) * 16), 16, 0, AUX);
  }
};

// Byte offset of chunk (row, c) inside a swizzled LDS tile.
template <int NC, Swz MODE> AAT_DEV int lds_chunk_off(int row, int c) {
  return (row * NC + swz<NC, MODE>(row, c)) * 16;
}

// ---------------------------------------------------------------------------------------------------
// LDS reads in MFMA operand layouts.
AAT_DEV h8 lds_read_h8(const char* p) { return *reinterpret_cast<const h8*>(p); }

// Transposing read: within each group of 16 lanes, source lane s points at 4 contiguous halfs of row
// s/4, column group s%4 of a 4-row x 16-column patch; destination lane i receives column i, rows 0..3.
AAT_DEV h4 lds_read_tr_h4(const char* p) {
  fp16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((AAT_AS3 fp16x4_t*)(p));
  h4 o;
  __builtin_memcpy(&o, &r, 8);
  return o;
}
AAT_DEV h8 cat_h4(h4 lo, h4 hi) {
  h8 r;
  r[0] = lo[0]; r[1] = lo[1]; r[2] = lo[2]; r[3] = lo[3];
  r[4] = hi[0]; r[5] = hi[1]; r[6] = hi[2]; r[7] = hi[3];
  return r;
}

// ---------------------------------------------------------------------------------------------------
// fp32 -> fp16 round-to-nearest-even, two at a time (v_cvt_pk_f16_f32).  The reference converts P, S,
// dS and every output with cutlass::NumericArrayConverter, which is RNE as well
// (reference: csrc/kernels/attention/regfuse/regfuse.h:298-301, retnet/bwd/bwd_colblock.h:69-78).
AAT_DEV h2 pack_rne(float a, float b) {
  f2v p = {a, b};
  return __builtin_convertvector(p, h2);
}
// Eight accumulator registers v0..v0+7 of a C tile -> one MFMA B/A operand.
AAT_DEV h8 pack8_rne(const f16v& c, int v0) {
  h8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    h2 p = pack_rne(c[v0 + 2 * i], c[v0 + 2 * i + 1]);
    r[2 * i] = p[0];
    r[2 * i + 1] = p[1];
  }
  return r;
}

// ---------------------------------------------------------------------------------------------------
// Exchange with lane^32 (v_permlane32_swap): the two lanes that share a query row in the S^T layout.
AAT_DEV float other_half(float x) {
  u2v r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  const float lo = __uint_as_float(r[0]), hi = __uint_as_float(r[1]);
  // r[0] holds the lower half's value in all lanes, r[1] the upper half's.
  return (threadIdx.x & 32) ? lo : hi;
}
AAT_DEV float pair_max(float x) {
  u2v r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
AAT_DEV float pair_sum(float x) {
  u2v r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

AAT_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
AAT_DEV float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

// ---------------------------------------------------------------------------------------------------
// Workgroup id -> tile id so that tiles sharing one (batch, head) -- and therefore one K/V stream --
// run on the same XCD and hit the same L2.  Hardware deals consecutive workgroup ids round-robin over
// the 8 XCDs; this undoes that when the grid is a multiple of 8.
AAT_DEV int xcd_remap(int wg, int grid) {
  constexpr int kXcd = 8;
  if (grid % kXcd != 0) return wg;
  return (wg % kXcd) * (grid / kXcd) + wg / kXcd;
}

// (batch*head, block) of a workgroup in a causal walk with T blocks per head.  A block's length grows
// linearly with its position in the head (row blocks: the last one is the longest; kv blocks of a
// column pass: the first one), and the chip holds only part of the grid at a time, so the order in which
// blocks are dealt out decides the tail of the launch.  Longest first *within each head* is not enough:
// the CUs that finish a head's short blocks early are handed the next head's longest ones.  The blocks of
// all heads that share an XCD are therefore dealt out in one sequence sorted by length, longest first,
// which lets every CU end up with about the same total (a head still stays on one XCD and one L2).
struct TileId {
  int bh, blk;
};
AAT_DEV TileId causal_tile(int wg, int grid, int T, bool last_is_longest) {
  const int tile = xcd_remap(wg, grid);
  const int per_xcd = grid / 8;
  int bh = tile / T, pos = tile % T;
  if (grid % 8 == 0 && per_xcd % T == 0) {
    const int heads = per_xcd / T;                // heads per XCD
    const int l = tile % per_xcd;
    bh = (tile / per_xcd) * heads + l % heads;
    pos = l / heads;
  }
  return {bh, last_is_longest ? T - 1 - pos : pos};
}

}  // namespace aat
