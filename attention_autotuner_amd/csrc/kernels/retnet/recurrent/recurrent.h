// RetNet recurrent form  S_n = a_n * S_{n-1} + k_n^T v_n,  out_n = q_n S_n  (fp32, per-position decay a).
//
// Same result as reference csrc/kernels/retnet/recurrent/recurrent.h:133-463 (a CUB BlockScan over
// (decay, k*v) pairs, one scan per (key dim, value dim) pair, launched by retnet_recurrent_fwd :427-463),
// same tensors: q, k [B, H, kdim, L], v, out [B, H, vdim, L] (sequence contiguous), decay [H, L].
//
// The scan is evaluated chunk by chunk on the fp32 matrix cores instead of element by element on the
// vector ALU.  For a chunk of 32 positions, with State = S at the end of the previous chunk:
//   S^T[m][n]  = sum_kd K[kd][m] Q[kd][n]                          (keys m x queries n)
//   P[m][n]    = S^T[m][n] * prod_{m<j<=n} a_j  (0 for m > n)      exact running products, no logarithms
//   O^T[vd][n] = p_n * sum_kd State[kd][vd] Q[kd][n] + sum_m V[vd][m] P[m][n],   p_n = prod_{j<=n} a_j
//   State[kd][vd] = A * State[kd][vd] + sum_m K[kd][m] w_m V[vd][m],   w_m = prod_{j>m} a_j, A = prod_j a_j
// which is 5 flops per (position, kd, vd) -- what the element-wise recurrence itself costs -- but at the
// MFMA rate.  No logarithms or divisions: zero and negative decays behave as in the recurrence.
//
// One block owns one (batch, head) and a slice of DVS value dims; wave w owns value dims [32w, 32w+32) of
// the slice: its State tiles (KD x 32, fp32, in registers for the whole sequence) and its rows of O^T.
// v_mfma_f32_32x32x2_f32, lane l, half h = l/32, column j = l%32:
//   A (32 x 2): lane holds A[j][h];  B (2 x 32): lane holds B[h][j];  C (32 x 32): lane holds C[8g+4h+e][j].
// The contraction index of a step is free as long as A and B agree, so step (g, e) is given the index
// 8g+4h+e: then the C registers of one product ARE the A or B operand of the next (State feeds
// State^T*Q, P feeds V*P) and no value ever changes lanes.
// S^T is split over the waves along kd (each wave contracts KD/waves key dims), the partial tiles are
// summed through LDS; every other product is private to its wave.
#pragma once
#include "kernels/utils/cdna4.h"
#include "kernels/utils/tile_ops.h"

namespace aat {

AAT_DEV f16v mfma_32x32x2_f32(float a, float b, f16v c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// ---------------------------------------------------------------------------------------------------
// LDS tile of ROWS x 32 floats (8 chunks of 16 bytes per row).  Row r sits at position pos(r) = r with
// bits 0 and 2 exchanged, chunk c of the row at position p in slot c ^ ((p >> 1) & 7).
//  * reads along the sequence (one dword per lane, lanes 0-31 one row, lanes 32-63 the row 4 below):
//    the two rows land on positions of different parity, i.e. on different halves of the 64 banks;
//  * reads across rows (one 16-byte chunk per lane, 16 consecutive rows per 256-byte LDS cycle): the
//    slot term is a bijection of the 16 positions onto the 16 slots.
AAT_DEV constexpr int rec_pos(int r) { return (r & ~5) | ((r & 1) << 2) | ((r >> 2) & 1); }
AAT_DEV constexpr int rec_slot(int p, int c) { return c ^ ((p >> 1) & 7); }
AAT_DEV constexpr int rec_off(int r, int col) {                       // byte offset of element (r, col)
  const int p = rec_pos(r);
  return p * 128 + rec_slot(p, col >> 2) * 16 + (col & 3) * 4;
}
constexpr bool rec_row_reads_conflict_free() {
  for (int r = 0; r < 32; ++r) {
    if (r & 4) continue;
    unsigned long long seen = 0;
    for (int l = 0; l < 64; ++l) {
      const int bank = (rec_off(r + 4 * (l >> 5), l & 31) >> 2) & 63;
      if (seen >> bank & 1ull) return false;
      seen |= 1ull << bank;
    }
  }
  return true;
}
constexpr bool rec_column_reads_conflict_free() {
  for (int r0 = 0; r0 < 32; r0 += 16)
    for (int c = 0; c < 8; ++c) {
      unsigned seen = 0;
      for (int i = 0; i < 16; ++i) {
        const int slot = (rec_off(r0 + i, 4 * c) >> 4) & 15;
        if (seen >> slot & 1u) return false;
        seen |= 1u << slot;
      }
    }
  return true;
}
static_assert(rec_row_reads_conflict_free() && rec_column_reads_conflict_free(),
              "both access patterns of the fp32 chunk tiles are free of LDS bank conflicts");

// ---------------------------------------------------------------------------------------------------
// Decay factors of one (head, chunk), computed once by retnet_recurrent_factors and shared by every
// batch entry and value slice.  Vector-ALU instructions do not overlap fp32 MFMAs on this hardware, so
// everything that depends on the decay alone is taken out of the main kernel.
//
// State is kept as T = State / lambda with a per-head scalar lambda (the product of the decays since
// the last rescale), so that a chunk's decay does not have to be multiplied into the KD x DVS state:
//   O^T = (p_n lambda) (T^T Q) + V P,      T += K diag(w / lambda') V^T,   lambda' = A lambda.
// When |lambda'| leaves [2^-40, 2^40] (or is zero) the record says so: the kernel then multiplies T by
// `scale` = A lambda once and lambda restarts at 1.
//   [0, 4096)     D[g][lane][e]   = prod_{m<j<=n} a_j for m = 8g+4h+e, n = lane%32, h = lane/32 (0 for m > n)
//   [4096, 4224)  W[h][g][e]      = w_m / lambda'      (w_m alone on a rescale)
//   [4224, 4352)  PNL[n]          = p_n lambda
//   [4352, 4360)  rescale flag (uint32), scale (float)
constexpr int kRecFactorBytes = 5120;
constexpr int kRecFactorW = 4096, kRecFactorPnl = 4224, kRecFactorFlag = 4352;

// decay [H][L] -> factors [H][L/32][kRecFactorBytes].  Grid H, kRecFactorThreads threads, 16 bytes of
// dynamic LDS per chunk.  The waves of a block share out the chunks of their head (products inside a
// chunk), one thread then walks lambda through the chunks, and the waves fold it into their records.
constexpr int kRecFactorThreads = 1024;
__global__ __launch_bounds__(kRecFactorThreads) void retnet_recurrent_factors(const float* __restrict__ decay,
                                                                              char* __restrict__ factors, int L) {
  extern __shared__ __align__(16) float fsm[];     // per chunk: A, lambda before the chunk, 1/lambda' (or 1), rescale flag
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 31, hi = lane >> 5, nchunk = L / 32;
  constexpr int kWavesF = kRecFactorThreads / 64;
  char* const recs = factors + (size_t)blockIdx.x * nchunk * kRecFactorBytes;
  for (int c = wave; c < nchunk; c += kWavesF) {
    const float* dg = decay + (size_t)blockIdx.x * L + c * 32;
    char* rec = recs + (size_t)c * kRecFactorBytes;
    float dsel[16], wsel[16];
    float d = 0.f, w = 1.f;
#pragma unroll
    for (int m = 31; m >= 0; --m) {     // exact running products, from the diagonal down
      if (m < 31) { d *= dg[m + 1]; w *= dg[m + 1]; }
      d = (m == n) ? 1.f : d;
      const int idx = (m >> 3) * 4 + (m & 3);
      if (m & 4) { dsel[idx] = d; wsel[idx] = w; }
      else { dsel[idx] = hi ? dsel[idx] : d; wsel[idx] = hi ? wsel[idx] : w; }
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f4v x = {dsel[4 * g], dsel[4 * g + 1], dsel[4 * g + 2], dsel[4 * g + 3]};
      *reinterpret_cast<f4v*>(rec + g * 1024 + lane * 16) = x;
      if (n == 0) {
        f4v y = {wsel[4 * g], wsel[4 * g + 1], wsel[4 * g + 2], wsel[4 * g + 3]};
        *reinterpret_cast<f4v*>(rec + kRecFactorW + hi * 64 + g * 16) = y;
      }
    }
    if (hi == 0) *reinterpret_cast<float*>(rec + kRecFactorPnl + n * 4) = d * dg[0];    // p_n
    if (lane == 0) fsm[4 * c] = w * dg[0];                                             // A
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float lam = 1.f;
    for (int c = 0; c < nchunk; ++c) {
      const float lam_new = fsm[4 * c] * lam;
      const float mag = __builtin_fabsf(lam_new);
      const bool rescale = !(mag >= 0x1p-40f && mag <= 0x1p40f);
      char* rec = recs + (size_t)c * kRecFactorBytes;
      *reinterpret_cast<uint32_t*>(rec + kRecFactorFlag) = rescale ? 1u : 0u;
      *reinterpret_cast<float*>(rec + kRecFactorFlag + 4) = lam_new;
      fsm[4 * c + 1] = lam;
      fsm[4 * c + 2] = rescale ? 1.f : 1.f / lam_new;
      lam = rescale ? 1.f : lam_new;
    }
  }
  __syncthreads();
  for (int c = wave; c < nchunk; c += kWavesF) {
    char* rec = recs + (size_t)c * kRecFactorBytes;
    if (lane < 32) {
      float* w = reinterpret_cast<float*>(rec + kRecFactorW + lane * 4);
      *w *= fsm[4 * c + 2];
    } else {
      float* p = reinterpret_cast<float*>(rec + kRecFactorPnl + (lane - 32) * 4);
      *p *= fsm[4 * c + 1];
    }
  }
}

template <int KD, int DVS>
struct RetRecurrent {
  static constexpr int kChunk = 32;                       // positions per step
  static constexpr int kWaves = DVS / 32;
  static constexpr int kThreads = kWaves * 64 + 64;        // the matrix waves plus one wave that moves the data
  static constexpr int kKB = KD / 32;                     // State tiles per wave
  static constexpr int kGroups = KD / 8;                  // groups of 8 key dims (one (h, e) sweep of a step)
  static constexpr int kGroupsPerWave = kGroups / kWaves; // share of one wave in the S^T contraction
  static constexpr int kKTile = KD * 128, kVTile = DVS * 128;
  static constexpr int kQOff = kKTile, kVOff = 2 * kKTile, kFOff = 2 * kKTile + kVTile;
  static constexpr int kStage = kFOff + kRecFactorBytes;  // K, Q, V tiles and the decay factors of one chunk
  static constexpr int kRed = kWaves * 4096;              // one partial S^T tile per wave
  static constexpr int kOutOff = 2 * kStage + kRed;       // per wave: its 32 x 32 output tile, staged for 16-byte stores
  static constexpr int kSmemBytes = kOutOff + kWaves * 4096;
  static_assert(KD % 32 == 0 && DVS % 64 == 0 && DVS <= 256, "tile shape");
  static_assert(kGroups % kWaves == 0, "the S^T contraction must split evenly over the waves");
  static_assert(kFOff + kRecFactorBytes <= 65536, "tile offsets go into the 16-bit offset field of the LDS reads");
  static_assert(kSmemBytes <= 160 * 1024, "LDS");
};

// LDS reads and stores issued by hand so that their waits can be counted: the compiler answers every
// dependency on an LDS load with lgkmcnt(0) while an LDS-DMA copy is in flight, and here one is in
// flight all the time.  LDS operations retire in order, so "at most N younger ones outstanding" is enough.
AAT_DEV float lds_read_f1_async(uint32_t base, int imm) {
  float v;
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(base), "i"(imm));
  return v;
}
template <int N, class V> AAT_DEV void lds_wait_younger_f(V& v) {
  static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit counter");
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(N));
}

// q, k: [B*H][kdim][L]; v, out: [B*H][vdim][L]; factors: output of retnet_recurrent_factors.  Contracts
// the first KD key dims (the reference's block_kdim, reference recurrent.h:290,427).  Grid (vdim / DVS, B*H).
// Compiled for two waves per SIMD's worth of registers (256): then every MFMA takes and leaves its
// operands in vector registers and nothing has to be moved between register classes.
//
// Waves 0 .. DVS/32-1 do the arithmetic; the last wave of the block only moves data: it issues every
// LDS-DMA copy of the next chunk and stores the previous chunk's output tiles from their LDS staging
// area.  An LDS-DMA or store instruction holds its wave for 16 to 50 cycles (thousands for a burst), and a
// matrix wave is the only one on its SIMD: whatever it spends issuing memory instructions the matrix core
// idles.  The data wave has nothing else to do.
template <int KD, int DVS>
__global__ __launch_bounds__(DVS * 2 + 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void retnet_recurrent_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
    const char* __restrict__ factors, float* __restrict__ out, int heads, int kdim, int vdim, int L) {
  using T = RetRecurrent<KD, DVS>;

  extern __shared__ __align__(16) char smem[];

  const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, hi = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bh = blockIdx.y, h = bh % heads;
  const int nchunk = L / T::kChunk;
  const char* qg = reinterpret_cast<const char*>(q + (size_t)bh * kdim * L);
  const char* kg = reinterpret_cast<const char*>(k + (size_t)bh * kdim * L);
  const char* vg = reinterpret_cast<const char*>(v + ((size_t)bh * vdim + (size_t)blockIdx.x * DVS) * L);
  const char* fg = factors + (size_t)h * nchunk * kRecFactorBytes;
  const int pitch = L * 4;
  // Output: a wave's O^T tile goes through LDS so that it leaves as four 16-byte-per-lane stores (8 rows
  // x 128 bytes each) instead of sixteen 4-byte ones.  Row r of the tile sits at position r ^ ((r>>2)&1):
  // the two rows a write covers (r, r+4) and the two rows a 16-lane read phase covers (2m, 2m+1) then
  // fall on different halves of the banks.
  const int orl = lane >> 3, occ = lane & 7;

  if (wave == T::kWaves) {
    // ================================ data wave =================================================
    // LDS-DMA of a tile of 128-byte rows: instruction i covers positions 8i .. 8i+7, lane l position
    // 8i + l/8, chunk slot l%8.  The source row is rec_pos(position), the source chunk the slot XOR the
    // position's slot term (whose high bit is the parity of i).  Every address below is a scalar base that
    // moves with the chunk plus a per-lane 32-bit offset computed here once: the loop of this wave must not
    // contain a single vector instruction -- a vector instruction has to find a gap between the fp32 MFMAs
    // of the matrix wave that shares the SIMD, and a copy that waits for one took 175 cycles to issue.
    constexpr int kTileOps = (KD > DVS ? KD : DVS) / 8;
    uint32_t toff[kTileOps];
#pragma unroll
    for (int i = 0; i < kTileOps; ++i)
      toff[i] = (uint32_t)((8 * i + rec_pos(orl)) * pitch + (occ ^ (((i & 1) << 2) | (orl >> 1))) * 16);
    const uint32_t lane16off = lane * 16;
    auto dma_one = [&](const char* g_uniform, uint32_t lane_off, char* lds) {   // written out: scalar base + lane offset form
      const uint64_t base = (uint64_t)(uintptr_t)g_uniform;
      const uint32_t dst = (uint32_t)(uintptr_t)(AAT_AS3 char*)lds;
      asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                   :: "v"(lane_off), "s"(base), "s"(dst) : "memory", "m0");
    };
    // K and Q are needed first (the partial S^T opens a chunk); V and the decay factors follow.
    auto dma_kq = [&](int c, int stage) {
      char* s = smem + stage * T::kStage;
      const size_t col = (size_t)c * T::kChunk * 4;
#pragma unroll
      for (int i = 0; i < KD / 8; ++i) dma_one(kg + col, toff[i], s + i * 1024);
#pragma unroll
      for (int i = 0; i < KD / 8; ++i) dma_one(qg + col, toff[i], s + T::kQOff + i * 1024);
    };
    auto dma_vf = [&](int c, int stage) {
      char* s = smem + stage * T::kStage;
#pragma unroll
      for (int i = 0; i < DVS / 8; ++i) dma_one(vg + (size_t)c * T::kChunk * 4, toff[i], s + T::kVOff + i * 1024);
      const char* f = fg + (size_t)c * kRecFactorBytes;
#pragma unroll
      for (int i = 0; i < kRecFactorBytes / 1024; ++i) dma_one(f + i * 1024, lane16off, s + T::kFOff + i * 1024);
    };
    // output tiles of chunk c: one per matrix wave, four 8-row groups each; all reads first, one wait, then
    // the stores back to back, each a scalar base plus one of 16 precomputed lane offsets
    uint32_t ooff[T::kWaves][4];
#pragma unroll
    for (int w = 0; w < T::kWaves; ++w)
#pragma unroll
      for (int i = 0; i < 4; ++i) ooff[w][i] = (uint32_t)(((32 * w + 8 * i + orl) * L + occ * 4) * 4);
    const char* const oread = smem + T::kOutOff + (orl ^ ((orl >> 2) & 1)) * 128 + occ * 16;
    float* const og = out + ((size_t)bh * vdim + (size_t)blockIdx.x * DVS) * L;
    auto store_chunk = [&](int c) {
      f4v x[T::kWaves][4];
#pragma unroll
      for (int w = 0; w < T::kWaves; ++w)
#pragma unroll
        for (int i = 0; i < 4; ++i) x[w][i] = *reinterpret_cast<const f4v*>(oread + w * 4096 + i * 1024);
      wait_lgkm0();
      const uint64_t base = (uint64_t)(uintptr_t)(og + (size_t)c * T::kChunk);
#pragma unroll
      for (int w = 0; w < T::kWaves; ++w)
#pragma unroll
        for (int i = 0; i < 4; ++i) asm volatile("global_store_dwordx4 %0, %1, %2" :: "v"(ooff[w][i]), "v"(x[w][i]), "s"(base) : "memory");
    };
    dma_kq(0, 0);
    dma_vf(0, 0);
    wait_vmcnt<0>();
    for (int c = 0; c < nchunk; ++c) {
      const bool more = c + 1 < nchunk;
      asm volatile("s_barrier" ::: "memory");          // chunk c is in LDS; the matrix waves are done with chunk c-1
      if (more) dma_kq(c + 1, (c + 1) & 1);
      if (c > 0) store_chunk(c - 1);                     // staged before this barrier, overwritten after the next one
      if (more) dma_vf(c + 1, (c + 1) & 1);
      asm volatile("s_barrier" ::: "memory");          // (the matrix waves' barrier in front of the S^T sum, late in the chunk)
      wait_vmcnt<0>();                                   // the next chunk has landed, the stores are out
    }
    asm volatile("s_barrier" ::: "memory");              // the last chunk's tiles are staged
    store_chunk(nchunk - 1);
    return;
  }

  // ================================ matrix waves ================================================
  char* const ost = smem + T::kOutOff + wave * 4096;
  char* const ow_even = ost + n * 4 + 5 * hi * 128;                         // write base for e even: position 4h + h
  char* const ow_odd = ost + n * 4 + (3 * hi + 1) * 128;                    // e odd: position 4h + (1 - h)

  // Per-lane LDS read addresses of the current stage (moved to the other stage at the end of a chunk).
  //  row read (row 8G+4h+e, column n): the slot term of the row is the compile-time constant
  //  sw(G, e) = 4(G&1) + 2(e&1) + (e>>1), folded into the lane part by XOR; the row goes into the offset.
  //  column read (16-byte chunk 2g+h of row n of a 32-row block): position and slot term are per lane.
  const uint32_t lds0 = lds_addr(smem);
  const uint32_t row_lane = hi * 128 + (n >> 2) * 16 + (n & 3) * 4;
  const int wave_rows = wave * T::kGroupsPerWave * 8;                 // first key dim of this wave's share of S^T
  const int wave_sw = 4 * ((wave * T::kGroupsPerWave) & 1);
  const int cp = rec_pos(n);
  constexpr int kNumBases = 8 + 8 + 4 + 4 + 4;
  uint32_t bases[kNumBases];
  uint32_t* const row4 = bases;            // [8]  State^T Q operand rows
  uint32_t* const row1 = bases + 8;        // [8]  this wave's rows of the S^T contraction
  uint32_t* const colb = bases + 16;       // [4]  K columns
  uint32_t* const colv = bases + 20;       // [4]  V columns of this wave's 32 value dims
  uint32_t& lane16 = bases[24];
  uint32_t& wbase = bases[25];
  uint32_t& pbase = bases[26];
  uint32_t& sbase = bases[27];
#pragma unroll
  for (int sw = 0; sw < 8; ++sw) {
    row4[sw] = lds0 + (row_lane ^ (sw << 4));
    row1[sw] = lds0 + wave_rows * 128 + (row_lane ^ ((sw ^ wave_sw) << 4));
  }
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    colb[g] = lds0 + cp * 128 + rec_slot(cp, 2 * g + hi) * 16;
    colv[g] = colb[g] + T::kVOff + wave * 4096;
  }
  lane16 = lds0 + lane * 16;
  wbase = lds0 + hi * 64;
  pbase = lds0 + n * 4;
  sbase = lds0;
  uint32_t redo[T::kWaves - 1];                                       // the other waves' partial tiles
#pragma unroll
  for (int t = 0; t < T::kWaves - 1; ++t) redo[t] = lds0 + 2 * T::kStage + ((wave + 1 + t) % T::kWaves) * 4096 + lane * 16;
  char* const red_mine = smem + 2 * T::kStage + wave * 4096 + lane * 16;

  f16v st[T::kKB];
#pragma unroll
  for (int i = 0; i < T::kKB; ++i) st[i] = zero16();

  // The LDS reads of a chunk form one stream, consumed in order, each issued kPF elements ahead.
  constexpr int kPF = 6, kRing = kPF + 1;
  constexpr int nS1 = 8 * T::kGroupsPerWave;              // K and Q row reads of the partial S^T
  constexpr int nS4 = 16 * T::kKB;                        // Q row reads of State^T Q
  constexpr int nRedG = T::kWaves;                        // per g: the other waves' partials, then D
  // Order after State^T Q: the State update comes first (it needs V, w and K only), the sum of the partial
  // S^T tiles, P and V P sit inside it, before its last 16 matrix instructions.  Whatever a vector phase
  // needs from the matrix pipe (O^T for its scaling, V P for the staging of the output tile) then left it a
  // thousand cycles earlier, and the barrier in front of the partial tiles comes late in the chunk.
  constexpr int jS4 = nS1, jFlag = jS4 + nS4, jV = jFlag + 1, jW = jV + 4, jK1 = jW + 4;
  constexpr int jRed = jK1 + 4 * (T::kKB - 1), jPnl = jRed + 4 * nRedG, jK2 = jPnl + 1;
  constexpr int nElem = jK2 + 4;

  auto chunk = [&](auto stage_tag, int c) {
    constexpr int S = decltype(stage_tag)::value;
    float fr[kRing];
    f4v vr[kRing];
    f16v sp = zero16(), oacc = zero16(), pm;
    f4v vt[4], wv[4];
    float ka = 0.f;

    auto issue = [&](auto jt) {
      constexpr int j = decltype(jt)::value, slot = j % kRing;
      if constexpr (j < nS1) {
        constexpr int i = j / 2, gg = i / 4, e = i % 4, p0 = 8 * gg + 4 * (e & 1) + (e & 2), sw = (p0 >> 1) & 7;
        fr[slot] = lds_read_f1_async(row1[sw], (j % 2 ? T::kQOff : 0) + p0 * 128);
      } else if constexpr (j < jFlag) {
        constexpr int jj = j - jS4, G = jj / 4, e = jj % 4, p0 = 8 * G + 4 * (e & 1) + (e & 2), sw = (p0 >> 1) & 7;
        fr[slot] = lds_read_f1_async(row4[sw], T::kQOff + p0 * 128);
      } else if constexpr (j == jFlag) {
        vr[slot] = lds_read_f4_async(sbase, T::kFOff + kRecFactorFlag);
      } else if constexpr (j < jW) {
        vr[slot] = lds_read_f4_async(colv[j - jV], 0);
      } else if constexpr (j < jK1) {
        vr[slot] = lds_read_f4_async(wbase, T::kFOff + kRecFactorW + (j - jW) * 16);
      } else if constexpr (j < jRed) {
        constexpr int kb = (j - jK1) / 4, g = (j - jK1) % 4;
        vr[slot] = lds_read_f4_async(colb[g], kb * 4096);
      } else if constexpr (j < jPnl) {
        constexpr int g = (j - jRed) / nRedG, t = (j - jRed) % nRedG;
        if constexpr (t < T::kWaves - 1) vr[slot] = lds_read_f4_async(redo[t], g * 1024);
        else vr[slot] = lds_read_f4_async(lane16, T::kFOff + g * 1024);
      } else if constexpr (j == jPnl) {
        fr[slot] = lds_read_f1_async(pbase, T::kFOff + kRecFactorPnl);
      } else {
        vr[slot] = lds_read_f4_async(colb[j - jK2], (T::kKB - 1) * 4096);
      }
    };

    auto consume = [&](auto jt) {
      constexpr int j = decltype(jt)::value, slot = j % kRing, younger = (nElem - 1 - j < kPF) ? nElem - 1 - j : kPF;
      if constexpr (j < nS1) {
        lds_wait_younger_f<younger>(fr[slot]);
        if constexpr (j % 2 == 0) ka = fr[slot];
        else sp = mfma_32x32x2_f32(ka, fr[slot], sp);
        if constexpr (j == nS1 - 1) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f4v x = {sp[4 * g], sp[4 * g + 1], sp[4 * g + 2], sp[4 * g + 3]};
            *reinterpret_cast<f4v*>(red_mine + g * 1024) = x;
          }
          asm volatile("" ::: "memory");     // the stores stay here, far ahead of the barrier that publishes them
        }
      } else if constexpr (j < jFlag) {
        constexpr int jj = j - jS4;
        lds_wait_younger_f<younger>(fr[slot]);
        oacc = mfma_32x32x2_f32(st[jj / 16][jj % 16], fr[slot], oacc);
      } else if constexpr (j == jFlag) {
        lds_wait_younger_f<younger>(vr[slot]);
        if (__builtin_amdgcn_readfirstlane(__float_as_uint(vr[slot][0])) != 0u) {   // lambda left its range: fold it into T
          const float sc = vr[slot][1];
#pragma unroll
          for (int kb = 0; kb < T::kKB; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) st[kb][i] *= sc;
        }
      } else if constexpr (j < jW) {
        lds_wait_younger_f<younger>(vr[slot]);
        vt[j - jV] = vr[slot];
      } else if constexpr (j < jK1) {
        lds_wait_younger_f<younger>(vr[slot]);
#pragma unroll
        for (int e = 0; e < 4; ++e) wv[j - jW][e] = vt[j - jW][e] * vr[slot][e];
      } else if constexpr (j < jRed) {
        constexpr int kb = (j - jK1) / 4, g = (j - jK1) % 4;
        lds_wait_younger_f<younger>(vr[slot]);
#pragma unroll
        for (int e = 0; e < 4; ++e) st[kb] = mfma_32x32x2_f32(vr[slot][e], wv[g][e], st[kb]);
      } else if constexpr (j < jPnl) {
        constexpr int g = (j - jRed) / nRedG, t = (j - jRed) % nRedG;
        lds_wait_younger_f<younger>(vr[slot]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (t < T::kWaves - 1) sp[4 * g + e] += vr[slot][e];
          else pm[4 * g + e] = sp[4 * g + e] * vr[slot][e];
        }
      } else if constexpr (j == jPnl) {
        lds_wait_younger_f<younger>(fr[slot]);
        // O^T = (p_n lambda) T^T Q + V P
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[i] *= fr[slot];
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int e = 0; e < 4; ++e) oacc = mfma_32x32x2_f32(vt[g][e], pm[4 * g + e], oacc);
      } else {
        constexpr int kb = T::kKB - 1, g = j - jK2;
        lds_wait_younger_f<younger>(vr[slot]);
#pragma unroll
        for (int e = 0; e < 4; ++e) st[kb] = mfma_32x32x2_f32(vr[slot][e], wv[g][e], st[kb]);
        if constexpr (j == nElem - 1) {
#pragma unroll
          for (int gg = 0; gg < 4; ++gg)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              *reinterpret_cast<float*>((e & 1 ? ow_odd : ow_even) + (8 * gg + (e & 2)) * 128) = oacc[4 * gg + e];
          asm volatile("" ::: "memory");     // staged before the barrier that hands it to the data wave
        }
      }
    };

    asm volatile("s_barrier" ::: "memory");   // chunk c is in LDS (the data wave waited for it); every wave is done with chunk c-1
    static_for<kPF>([&](auto jt) { issue(jt); });
    sched_fence();
    static_for<nElem>([&](auto jt) {
      constexpr int j = decltype(jt)::value;
      if constexpr (j + kPF < nElem) {
        // the partial tiles were stored long before (LDS operations retire in order and younger reads
        // have been waited for), so a bare barrier is enough before the first read of another wave's tile
        if constexpr (j + kPF == jRed) asm volatile("s_barrier" ::: "memory");
        issue(std::integral_constant<int, j + kPF>{});
      }
      consume(jt);
      sched_fence();
    });
#pragma unroll
    for (int i = 0; i < kNumBases; ++i) bases[i] += (S == 0) ? T::kStage : -T::kStage;
  };

  for (int c = 0; c < nchunk; c += 2) {
    chunk(std::integral_constant<int, 0>{}, c);
    if (c + 1 < nchunk) chunk(std::integral_constant<int, 1>{}, c + 1);
  }
  wait_lgkm0();
  asm volatile("s_barrier" ::: "memory");     // the last chunk's output tiles are staged: the data wave stores them
}

}  // namespace aat
