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
//  * the running max is lazy (softmax.h);
//  * two schedules: the plain one walks Bc-wide tiles (scores, softmax, PV, in that order); the
//    pipelined one works in 32-row units and issues the MFMAs of the NEXT unit's scores between the
//    exponentials of the current unit, so the matrix and vector pipes overlap inside one wave;
//  * softmax scale and causal masking are runtime arguments (the reference hard-codes 0.125 at :50 and
//    has the causal bound commented out at :59-61).
#pragma once
#include <type_traits>

#include "../../utils/cdna4.h"
#include "../../utils/softmax.h"
#include "../../utils/tile_ops.h"

#ifndef AAT_PF
#define AAT_PF 2
#endif
#ifdef AAT_NOPRIO
#define AAT_SETPRIO(x)
#else
#define AAT_SETPRIO(x) __builtin_amdgcn_s_setprio(x)
#endif

namespace aat {

template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV>
struct AttnFwdRegfuse {
  static constexpr int NW = Nthreads / kWave;   // waves per block
  static constexpr int WM = Br / NW;            // query rows per wave
  static constexpr int RT = WM / 32;            // 32-row groups per wave
  static constexpr int NT = Bc / 32;            // score tiles (units) along kv
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
  static constexpr int kUnitK = 32 * Kd * 2, kUnitV = 32 * D * 2;   // bytes of one 32-row unit
  static constexpr int kOStride = D * 2 + 16;   // epilogue staging row stride (bytes)
  static constexpr int kMainBytes = NSK * kKBytes + NSV * kVBytes;
  static constexpr int kEpiBytes = Br * kOStride;
  static constexpr int kSmemBytes = kMainBytes > kEpiBytes ? kMainBytes : kEpiBytes;
  static constexpr int kSmemBytesSplit = kMainBytes;   // the partial outputs of a kv split are stored without staging
  // Persistent blocks (PERSIST) stage their output tiles where the copies of the next row block's first kv
  // tile do not land: behind the K/V buffers as far as the LDS budget of a block goes, then in the second K
  // and the second V buffer (the last kv tile of a row block has parity 1, the prefetch goes to parity 0).
  static constexpr int kStageWave = WM * kOStride;
  template <int WPE> struct Persist {
    static constexpr int kBlocksByRegs = (WPE * 4) / NW > 0 ? (WPE * 4) / NW : 1;   // resident blocks the registers allow
    static constexpr int kBudget = (160 * 1024 / kBlocksByRegs) & ~2047;            // whole allocation units
    static constexpr int kWant = kMainBytes + NW * kStageWave;
    static constexpr int kFit = kWant < kBudget ? kWant : kBudget;
    static constexpr int kSmemBytes = kFit > kMainBytes ? kFit : kMainBytes;
    static constexpr int kInSpare = (kSmemBytes - kMainBytes) / kStageWave;
    static constexpr int kInK = kKBytes / kStageWave, kInV = kVBytes / kStageWave;
    // WPE >= 2: the next row block's Q fragments are requested into live registers behind the compiler's back.  With the
    // unified register file of two or more waves per SIMD those registers stay where they are; a wave that owns the
    // split file (256 vector + 256 accumulation registers) has its fragments moved between the two classes at the
    // compiler's discretion, and a copy made before the data has arrived carries stale values.
    static constexpr bool kOk = NSK == 2 && NSV == 2 && WPE >= 2 && kInSpare + kInK + kInV >= NW;
    static constexpr bool kSharesBuffers = kInSpare < NW;   // then every wave must be done with the last tile first
    static constexpr int kOutputStores = RT * D / 16;       // 16-byte-per-lane store instructions of one output tile
    static_assert(kOutputStores + RT < 64, "vmcnt is a 6-bit counter");
    AAT_DEV static int stage_offset(int wave) {
      if (wave < kInSpare) return kMainBytes + wave * kStageWave;
      if (wave < kInSpare + kInK) return kKBytes + (wave - kInSpare) * kStageWave;
      return NSK * kKBytes + kVBytes + (wave - kInSpare - kInK) * kStageWave;
    }
  };
  // The pipelined schedule copies K in whole 32-row units.
  static constexpr bool kPipeOk = NSK == 2 && NSV == 2 && KDma::kRegular && KDma::kRowsPerIter <= 32 &&
                                  32 % KDma::kRowsPerIter == 0;
  static constexpr int kKInstrPerUnit = KDma::kRegular ? 32 / (KDma::kRowsPerIter > 32 ? 32 : KDma::kRowsPerIter) : 0;
};

// Walk the kv tiles of a block two at a time (buffer parity 0, then 1).  Tiles [0, n_full) run the
// unmasked body; with CAUSAL the rest run the masked body.  n_full is even, so both loops start on
// parity 0 and every tile body is instantiated exactly once per (parity, masked) pair.
template <bool CAUSAL, class F> AAT_DEV void run_tiles(F& tile, int n_full, int n_tiles) {
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  const int n_plain = CAUSAL ? n_full : n_tiles;
  for (int j = 0; j < n_plain; j += 2) {
    tile(j, P0{}, std::false_type{});
    if (j + 1 < n_plain) tile(j + 1, P1{}, std::false_type{});
  }
  if constexpr (CAUSAL) {
    for (int j = n_full; j < n_tiles; j += 2) {
      tile(j, P0{}, std::true_type{});
      if (j + 1 < n_tiles) tile(j + 1, P1{}, std::true_type{});
    }
  }
}

// lse may be null.  When non-null it receives the natural-log-sum-exp of the scaled scores per row.
// PIPE selects the software-pipelined schedule (needs two K and two V buffers).  CAUSAL is a
// compile-time switch so that the non-causal kernel carries no masking code at all; in the causal
// kernel the tiles the diagonal cannot touch still run the unmasked tile body.
//
// SPLIT: the kv range is cut into gridDim.y equal parts (few query rows, long kv: not enough row
// blocks to fill the chip).  Part s handles kv tiles [s, s+1) * n_tiles / parts and writes its own
// normalised output (fp32) and log-sum-exp to part_o / part_lse, laid out [part][B*H*S_q][D] and
// [part][B*H*S_q]; attn_split_merge combines them.  o and lse are not touched.
//
// PERSIST: the grid is as many blocks as the chip holds at once and block b works through row blocks
// b, b + gridDim.x, ... of the n_items = B*H*S_q/Br there are.  A block that is alone on its CU otherwise
// pays for every row block the launch of a new block, the first trip to memory for Q, K and V with nothing
// to overlap it, and the drain of the output stores: 5.7 us of the 66 us a 256-row block of the 2048 x 2048
// problem takes.  Here the last kv tile of a row block requests tile 0 of the next one (K, V into the
// buffers of the other parity, Q into the fragment registers the moment the last scores are done), the
// output tile is staged where those copies do not land, and the first tile of the next row block waits for
// the copies only: memory operations complete in order, so "at most as many outstanding as stores were issued
// after them" leaves the stores in flight.  Needs two K and two V buffers and an even number of kv tiles (the
// buffer parity must wrap); plain schedule, non-causal, unsplit.
template <int Kd, int D, int Br, int Bc, int Nthreads, int NSK, int NSV, int WPE = 1, int BU = Bc, bool PIPE = false,
          bool CAUSAL = false, bool SPLIT = false, bool PERSIST = false, bool PAIR = false>
__global__ void __launch_bounds__(Nthreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
flashattn_fwd_regfuse(const half_t* __restrict__ q, const half_t* __restrict__ k,
                      const half_t* __restrict__ v, half_t* __restrict__ o, float* __restrict__ lse,
                      int H, int seq_k, int seq_q, float softmax_scale, float* __restrict__ part_o = nullptr,
                      float* __restrict__ part_lse = nullptr, int n_items = 0) {
  using T = AttnFwdRegfuse<Kd, D, Br, Bc, Nthreads, NSK, NSV>;
  constexpr int RT = T::RT, NT = T::NT, KS = T::KS, DT = T::DT, NCK = T::NCK, NCV = T::NCV, WM = T::WM, NW = T::NW;
  constexpr int PF = AAT_PF;                     // operand prefetch distance, in MFMA steps
  // Plain schedule: a kv tile of Bc rows (one copy, one barrier) is worked through in NU units of BU rows, each
  // scores -> softmax -> PV, so the live score tile is RT * BU / 32 accumulator blocks whatever Bc is.
  constexpr int NU = Bc / BU, NTU = BU / 32;
  static_assert(Bc % BU == 0 && BU % 32 == 0, "a kv tile is a whole number of units of whole 32-row score tiles");
  static_assert(NU == 1 || (NSK == 2 && NSV == 2), "units inside a tile: no barrier between the contractions, two K and two V buffers");
  static_assert(NU == 1 || !PIPE, "the pipelined schedule has its own 32-row units");
  // Where the output accumulators, the Q fragments and one unit's scores leave fewer than 40 of a wave's registers,
  // the operand addresses of all contraction steps are derived from one register each (tile_ops.h: XA).
  constexpr bool XA = WPE >= 2 && RT * (DT * 16 + KS * 4 + NTU * 16) + 40 > 512 / WPE;
  // Causal, two 32-row groups per wave: wave w owns groups w and 2 NW - 1 - w of the block's 2 NW, an early and a late
  // one.  In the tiles the diagonal crosses a group needs the kv rows up to its own, so with contiguous rows the last
  // wave works through the whole diagonal region while the first is done after one unit and waits at every barrier;
  // dealt out this way every wave has 2 NW + 1 group-units to do there.  A unit the late group sees and the early one
  // does not runs the contractions for the late group alone.
  constexpr bool ILV = CAUSAL && RT == 2 && !PIPE && NSK == 2 && NSV == 2;
  static_assert(!PIPE || T::kPipeOk, "the pipelined schedule needs 2+2 buffers and unit-aligned K copies");
  static_assert(!(SPLIT && CAUSAL), "kv splitting is for non-causal problems");
  using TP = typename T::template Persist<WPE>;
  static_assert(!PERSIST || (!PIPE && !CAUSAL && !SPLIT && TP::kOk), "persistent blocks: plain schedule, 2+2 buffers, room to stage the output");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* const kbuf = smem;
  char* const vbuf = smem + NSK * T::kKBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, h = lane >> 5;

  const int Tr = seq_q / Br;
  TileDma<Bc, NCK, Nthreads, Swz::Rows16, 0, XA> kdma;
  TileDma<Bc, NCV, Nthreads, Swz::Rows4, 0, XA> vdma;
  kdma.init(tid);
  vdma.init(tid);
  const int wave_base = wave * 64;

  h8 qf[RT][KS];
  uint32_t kaddr[KS], vaddr[DT];                 // this lane's operand addresses inside buffer 0
  {
    int koff[KS], voff[DT];
    k_frag_offsets<KS, NCK>(koff, n, h);
    v_frag_offsets<DT, NCV>(voff, lane);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds_addr(kbuf + koff[ks]);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vaddr[dt] = lds_addr(vbuf + voff[dt]);
  }

  const float c2 = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, softmax_scale * kLog2e)));   // wave-uniform: a scalar register
  const int diag = seq_k - seq_q;               // kv index allowed for query i is <= i + diag

  // One pass per row block: a single one unless PERSIST -- or PAIR (a variant of the causal kernel): then the grid is half
  // the row blocks and block p of a head walks row block Tr-1-p and then row block p.  The two lengths add up to the same
  // for every p, so every workgroup does the same amount of work whatever order the dispatcher hands them out in, and
  // the workgroups of a head run side by side on one XCD and share its K/V stream in L2 (dealing single row blocks out
  // longest-first over all heads of an XCD balances as well, but interleaves sixteen heads in every L2).
  bool prefetched = false;                      // Q fragments and kv tile 0 of this row block were requested by the previous pass
  static_assert(!PAIR || (CAUSAL && !PERSIST && !SPLIT), "pairs of row blocks: the causal walk");
  int pass = 0;
  for (int vb = blockIdx.x;; vb += gridDim.x) {
    const int tile = PERSIST ? xcd_remap(vb, n_items) : xcd_remap(vb, (int)gridDim.x);
    int bh = tile / Tr, rb = tile % Tr;
    if constexpr (CAUSAL) {
      if constexpr (PAIR) {
        const int half = Tr / 2;
        bh = tile / half;
        rb = pass == 0 ? Tr - 1 - tile % half : tile % half;
      } else {                                    // long rows first, over all heads of the XCD
        const TileId t = causal_tile(vb, (int)gridDim.x, Tr, true);
        bh = t.bh;
        rb = t.blk;
      }
    }
    const int q0 = rb * Br;
    int n_tiles = seq_k / Bc;
    int n_full = n_tiles;                         // tiles [0, n_full) are visible to every row of the block
    if constexpr (CAUSAL) {
      const int last = q0 + Br - 1 + diag;        // last visible kv index for this block
      const int lim = last < 0 ? 0 : last / Bc + 1;
      n_tiles = lim < n_tiles ? lim : n_tiles;
      const int full = (q0 + diag + 1) / Bc;
      n_full = full < 0 ? 0 : (full < n_tiles ? full : n_tiles);
      n_full &= ~1;                               // keep the masked loop on an even tile: buffer parity 0
    }

    int tile0 = 0;                                // first kv tile of this block's range
    if constexpr (SPLIT) {
      const int per = n_tiles / (int)gridDim.y;   // the launcher guarantees divisibility
      tile0 = (int)blockIdx.y * per;
      n_tiles = per;
      n_full = per;
    }
    const char* kg = reinterpret_cast<const char*>(k + ((size_t)bh * seq_k + (size_t)tile0 * Bc) * Kd);
    const char* vg = reinterpret_cast<const char*>(v + ((size_t)bh * seq_k + (size_t)tile0 * Bc) * D);

    // first row of the wave's first 32-row group inside the block, and the distance to its second group
    const int wrow0 = ILV ? 32 * wave : wave * WM;
    const int group_rows = ILV ? 32 * (2 * NW - 1 - 2 * wave) : 32;
    if (!prefetched) load_q_frags<RT, KS, Kd>(qf, q + ((size_t)bh * seq_q + q0 + wrow0 + n) * Kd + 8 * h, group_rows);
    // PERSIST: where the next row block of this block starts (tile numbers map to (head, row block) as above)
    const int vb_next = vb + (int)gridDim.x;
    const bool has_next = PERSIST && vb_next < n_items;
    const int tile_next = has_next ? xcd_remap(vb_next, n_items) : tile;
    const size_t bh_next = (size_t)(tile_next / Tr), q0_next = (size_t)(tile_next % Tr) * Br;
    const char* const kg_next = reinterpret_cast<const char*>(k + bh_next * seq_k * Kd);
    const char* const vg_next = reinterpret_cast<const char*>(v + bh_next * seq_k * D);
    const half_t* const q_next = q + (bh_next * seq_q + q0_next + wave * WM + n) * Kd + 8 * h;
    f16v oacc[RT][DT];
    float m_run[RT], l_run[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      m_run[rt] = -INFINITY;
      l_run[rt] = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) oacc[rt][dt] = zero16();
    }
    const int q_lim0 = q0 + wrow0 + n + diag;       // last kv index row n of row group 0 may see

    if constexpr (!PIPE) {
      // ============================ plain schedule =================================================
      if (n_tiles > 0 && !prefetched) {
        kdma.issue(kg, kbuf, wave_base);
        if constexpr (NSV == 2) vdma.issue(vg, vbuf, wave_base);
      }
      if (!prefetched) wait_vmcnt0_visible();        // the Q fragments are in (cdna4.h); tile 0 is waited for next anyway
      // `parity_tag` carries j & 1 as a compile-time value so that every LDS address of the tile is a
      // per-lane constant plus an immediate.
      auto kv_tile = [&](const int j, auto parity_tag, auto masked_tag) {
        constexpr int PAR = decltype(parity_tag)::value;
        constexpr bool MASKED = decltype(masked_tag)::value;   // the causal diagonal may cross this tile
        char* const vcur = vbuf + (NSV == 2 ? PAR * T::kVBytes : 0);
        const bool more = (j + 1 < n_tiles);
        if constexpr (WPE == 1) {
          // Above 256 registers the file is split into 256 vector and 256 accumulation registers: keep the
          // output accumulators in the accumulation half and the Q fragments in the vector half, or the
          // allocator parks Q there and copies four registers back in front of every MFMA.
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) asm volatile("" : "+a"(oacc[rt][dt]));
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[rt][ks]));
          }
        }

        // (A) K_j (and with two V buffers V_j) has landed; every wave is past iteration j-1.
        if (PERSIST && j == 0 && prefetched) {     // the previous row block's output stores stay in flight
          if (lse != nullptr) wait_vmcnt<TP::kOutputStores + RT>();
          else wait_vmcnt<TP::kOutputStores>();
        } else {
          wait_vmcnt<0>();
        }
        block_sync();
        if constexpr (NSV == 1) vdma.issue(vg + (size_t)j * T::kVBytes, vcur, wave_base);
        if (more) {
          if constexpr (NSK == 2) kdma.issue(kg + (size_t)(j + 1) * T::kKBytes, kbuf + (PAR ^ 1) * T::kKBytes, wave_base);
          if constexpr (NSV == 2) vdma.issue(vg + (size_t)(j + 1) * T::kVBytes, vbuf + (PAR ^ 1) * T::kVBytes, wave_base);
        }
        if constexpr (PERSIST) {
          if (!more && has_next) {                 // tile 0 of the next row block, into the buffers it will look in
            kdma.issue(kg_next, kbuf + (PAR ^ 1) * T::kKBytes, wave_base);
            vdma.issue(vg_next, vbuf + (PAR ^ 1) * T::kVBytes, wave_base);
          }
        }

        // A wave none of whose rows sees any kv row of a unit (above the diagonal) only keeps the block's copies
        // and barriers going: its P would be all zeros, which changes neither O nor l nor the maximum.
        // The matrix phases run at a raised wave priority: with two or three waves on the SIMD the one that has
        // MFMAs to issue goes first and the others' softmax arithmetic fills the gaps, not the other way round
        // (causal forward at three waves per SIMD: -1.4 %; nothing at two).
        static_for<NU>([&](auto unit_tag) {
          constexpr int U = decltype(unit_tag)::value;
          const int kv0 = j * Bc + U * BU;           // first kv row of the unit
          if constexpr (ILV) {
            // One body for both row groups; in a unit the early group no longer sees (and the late one does) its
            // MFMAs, its softmax step and its packing are branched around one by one.
            bool on0 = true, on1 = true;
            if constexpr (MASKED) {
              const int last_early = q0 + wrow0 + 31 + diag;            // last kv row the early group sees
              on0 = kv0 <= last_early;
              on1 = kv0 <= last_early + group_rows;
            }
            if (on1) {
              f16v sacc[RT][NTU];
              AAT_SETPRIO(2);
              qk_gemm_steps<RT, NTU, KS, NCK, PF, false, XA, MASKED && XA>(sacc, qf, kaddr, PAR * T::kKBytes + U * NTU * T::kUnitK, [](int) {}, on0);
              AAT_SETPRIO(0);
#pragma unroll
              for (int rt = 0; rt < RT; ++rt) {
                if (rt != 0 || on0 || !(MASKED && XA)) {
                  const int q_lim = q_lim0 + rt * group_rows;
                  // only the unit the group's own diagonal runs through has anything to mask (wave-uniform)
                  const bool crosses = MASKED && kv0 + BU - 1 > q0 + wrow0 + rt * group_rows + diag;
                  if (crosses) causal_mask<NTU>(sacc[rt], kv0, q_lim, h);
                  const float mc = lazy_max_step<NTU, DT>(sacc[rt], m_run[rt], l_run[rt], oacc[rt], c2);
                  exp_tile<NTU, XA>(sacc[rt], c2, mc);
                  if (crosses) zero_masked<NTU>(sacc[rt], kv0, q_lim, h);
                }
              }
              h8 pf[RT][NTU][2];
              AAT_SETPRIO(2);
              pv_gemm_steps<RT, NTU, DT, NCV, PF, false, XA, MASKED && XA>(oacc, pf, vaddr, PAR * T::kVBytes + U * NTU * T::kUnitV, [&](int g) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                  if (rt != 0 || on0 || !(MASKED && XA)) pack_p_group<NTU, XA>(pf[rt], sacc[rt], g, l_run[rt]);
                }
              }, on0);
              AAT_SETPRIO(0);
            }
            return;
          }
          bool wave_sees = true;
          if constexpr (MASKED) wave_sees = kv0 <= q0 + wave * WM + WM - 1 + diag;

          f16v sacc[RT][NTU];
          if (wave_sees) {
            AAT_SETPRIO(2);
            qk_gemm_steps<RT, NTU, KS, NCK, PF, false, XA>(sacc, qf, kaddr, (NSK == 2 ? PAR * T::kKBytes : 0) + U * NTU * T::kUnitK, [](int) {});
            AAT_SETPRIO(0);
          }
          if constexpr (PERSIST && U == NU - 1) {
            if (!more && has_next) load_q_frags_async<RT, KS, Kd>(qf, q_next);   // the last scores of this row block are done; waited for at (A)
          }
          if (wave_sees) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
              if constexpr (MASKED) causal_mask<NTU>(sacc[rt], kv0, q_lim0 + rt * 32, h);
              const float mc = lazy_max_step<NTU, DT>(sacc[rt], m_run[rt], l_run[rt], oacc[rt], c2);
              exp_tile<NTU, XA>(sacc[rt], c2, mc);
              if constexpr (MASKED) zero_masked<NTU>(sacc[rt], kv0, q_lim0 + rt * 32, h);
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
          if (wave_sees) {
            h8 pf[RT][NTU][2];
            AAT_SETPRIO(2);
            pv_gemm_steps<RT, NTU, DT, NCV, PF, false, XA>(oacc, pf, vaddr, (NSV == 2 ? PAR * T::kVBytes : 0) + U * NTU * T::kUnitV, [&](int g) {
#pragma unroll
              for (int rt = 0; rt < RT; ++rt) pack_p_group<NTU, XA>(pf[rt], sacc[rt], g, l_run[rt]);   // per-lane partial sums
            });
            AAT_SETPRIO(0);
          }
        });
      };
      run_tiles<CAUSAL>(kv_tile, n_full, n_tiles);
    } else {
      // ============================ pipelined schedule =============================================
      // The unit of work is 32 kv rows.  While unit u is exponentiated, the MFMAs of unit u+1's scores
      // run underneath; then O += V_u^T P_u runs with the fp16 packing of P_u underneath.  Two score
      // tiles are live (current, next).
      //
      // K is copied in Bc-row tiles that are SHIFTED by one unit against the V tiles: K copy j holds kv
      // rows [j*Bc + 32, (j+1)*Bc + 32), exactly the units whose scores are computed during iteration j
      // (units 1..NT-1 of tile j and unit 0 of tile j+1).  So iteration j reads K buffer j&1 only, while
      // copy j+1 streams into the other one; V tile j is read from V buffer j&1 while V_{j+1} streams
      // in.  One barrier per Bc rows.  Rows [0, 32) are fetched on their own in the prologue.
      constexpr int KI = T::kKInstrPerUnit;        // DMA instructions per 32 rows of K
      f16v sbuf[2][RT][1];
      auto issue_k_copy = [&](int jj, char* dst) { // K copy jj; the last one stops at the end of the range
        const char* src = kg + (size_t)jj * T::kKBytes + T::kUnitK;
        if (jj + 1 < n_tiles) kdma.issue(src, dst, wave_base);
        else kdma.template issue_part<0, (NT - 1) * KI>(src, dst, wave_base);
      };
      if (n_tiles > 0) {
        kdma.template issue_part<0, KI>(kg, kbuf + T::kKBytes + (NT - 1) * T::kUnitK, wave_base);   // rows [0, 32)
        issue_k_copy(0, kbuf);
        vdma.issue(vg, vbuf, wave_base);
        wait_vmcnt<0>();
        block_sync();
        qk_gemm_steps<RT, 1, KS, NCK, PF>(sbuf[0], qf, kaddr, T::kKBytes + (NT - 1) * T::kUnitK, [](int) {});
      }
      auto kv_tile = [&](const int j, auto parity_tag, auto masked_tag) {
        constexpr int PAR = decltype(parity_tag)::value;
        constexpr bool MASKED = decltype(masked_tag)::value;
        const bool last_tile = (j + 1 >= n_tiles);
        if constexpr (WPE == 1) {
          // Above 256 registers the file is split into 256 vector and 256 accumulation registers: keep the
          // output accumulators in the accumulation half and the Q fragments in the vector half, or the
          // allocator parks Q there and copies four registers back in front of every MFMA.
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) asm volatile("" : "+a"(oacc[rt][dt]));
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[rt][ks]));
          }
        }
        // K copy j and V_j have landed; every wave finished iteration j-1 (frees the other buffers).
        wait_vmcnt<0>();
        block_sync();
        if (!last_tile) {
          issue_k_copy(j + 1, kbuf + (PAR ^ 1) * T::kKBytes);
          vdma.issue(vg + (size_t)(j + 1) * T::kVBytes, vbuf + (PAR ^ 1) * T::kVBytes, wave_base);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const int cur = (PAR * NT + t) & 1;                        // which score buffer holds unit (j, t)
          auto& scur = sbuf[cur];
          auto& snext = sbuf[cur ^ 1];
          const int kv0 = j * Bc + 32 * t;
          float mc[RT];
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            if constexpr (MASKED) causal_mask<1>(scur[rt], kv0, q_lim0 + rt * 32, h);
            mc[rt] = lazy_max_step<1, DT>(scur[rt], m_run[rt], l_run[rt], oacc[rt], c2);
          }
          constexpr int kPerStep = (16 + KS - 1) / KS;               // exponentials per MFMA step
          if (t + 1 < NT || !last_tile) {
            // scores of the next unit: slot t of K buffer PAR
            qk_gemm_steps<RT, 1, KS, NCK, PF>(snext, qf, kaddr, PAR * T::kKBytes + t * T::kUnitK, [&](int step) {
#pragma unroll
              for (int rt = 0; rt < RT; ++rt) exp_range<1>(scur[rt], step * kPerStep, kPerStep, c2, mc[rt]);
            });
          } else {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) exp_tile<1>(scur[rt], c2, mc[rt]);
          }
          if constexpr (MASKED) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) zero_masked<1>(scur[rt], kv0, q_lim0 + rt * 32, h);
          }
          h8 pf[RT][1][2];
          pv_gemm_steps<RT, 1, DT, NCV, PF>(oacc, pf, vaddr, PAR * T::kVBytes + t * T::kUnitV, [&](int g) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) pack_p_group<1>(pf[rt], scur[rt], g, l_run[rt]);
          });
        }
      };
      run_tiles<CAUSAL>(kv_tile, n_full, n_tiles);
    }

    // ---- epilogue: normalise, round, store -------------------------------------------------------
    if constexpr (!PERSIST) {
      wait_vmcnt<0>();
      block_sync();                                // every wave is done with the K/V buffers
    } else if constexpr (TP::kSharesBuffers) {
      block_sync();                                // every wave is done with the parity-1 buffers
    }
    float inv[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const float l_tot = pair_sum(l_run[rt]);
      inv[rt] = l_tot > 0.f ? fast_rcp(l_tot) : 0.f;
      const size_t row = (size_t)bh * seq_q + q0 + wrow0 + rt * group_rows + n;
      const float row_lse = l_tot > 0.f ? m_run[rt] * softmax_scale + __logf(l_tot) : -INFINITY;
      if constexpr (SPLIT) {
        if (h == 0) part_lse[(size_t)blockIdx.y * gridDim.x * Br + row] = row_lse;   // gridDim.x * Br = B*H*S_q
      } else {
        if (lse != nullptr && h == 0) lse[row] = row_lse;
      }
    }
    if constexpr (SPLIT) {
      const size_t rows_total = (size_t)gridDim.x * Br;
      store_o_rows_f32<RT, DT, D>(oacc, inv, part_o + ((size_t)blockIdx.y * rows_total + (size_t)bh * seq_q + q0 + wave * WM) * D, lane);
    } else if constexpr (PERSIST) {
      store_o_tile<RT, DT, D, T::kOStride>(oacc, inv, smem + TP::stage_offset(wave),
                                           o + ((size_t)bh * seq_q + q0 + wave * WM) * D, lane);
    } else {
      // transposed through LDS for 16-byte coalesced stores
      store_o_tile<RT, DT, D, T::kOStride>(oacc, inv, smem + wave * WM * T::kOStride,
                                           o + ((size_t)bh * seq_q + q0 + wrow0) * D, lane, group_rows);
    }
    if constexpr (PAIR) {
      if (pass == 0) {
        pass = 1;
        vb -= (int)gridDim.x;                      // the same workgroup id again
        block_sync();                              // every wave has read its output tile out of the staging area
        continue;
      }
    }
    if (!has_next) break;
    prefetched = true;
  }
}

// Combine the parts of a kv split: O = sum_s exp(lse_s - lse) O_s with lse = log sum_s exp(lse_s).
// One thread per (row, 8 output columns); HBM-bound.
template <int D>
__global__ void __launch_bounds__(256)
attn_split_merge(const float* __restrict__ part_o, const float* __restrict__ part_lse, half_t* __restrict__ o,
                 float* __restrict__ lse, int rows, int parts) {
  constexpr int kChunks = D / 8;
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (size_t)rows * kChunks) return;
  const size_t row = idx / kChunks;
  const int c = (int)(idx % kChunks);
  float m = -INFINITY;
  for (int s = 0; s < parts; ++s) m = fmaxf(m, part_lse[(size_t)s * rows + row]);
  const float m_use = (m == -INFINITY) ? 0.f : m;
  float wsum = 0.f, acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  for (int s = 0; s < parts; ++s) {
    const float w = __expf(part_lse[(size_t)s * rows + row] - m_use);
    wsum += w;
    const f4v a = *reinterpret_cast<const f4v*>(part_o + ((size_t)s * rows + row) * D + c * 8);
    const f4v b = *reinterpret_cast<const f4v*>(part_o + ((size_t)s * rows + row) * D + c * 8 + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[e] += w * a[e];
      acc[4 + e] += w * b[e];
    }
  }
  const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
  h8 out;
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    const h2 pr = pack_rne(acc[e] * inv, acc[e + 1] * inv);
    out[e] = pr[0];
    out[e + 1] = pr[1];
  }
  *reinterpret_cast<h8*>(o + row * D + c * 8) = out;
  if (lse != nullptr && c == 0) lse[row] = wsum > 0.f ? m_use + __logf(wsum) : -INFINITY;
}

}  // namespace aat
