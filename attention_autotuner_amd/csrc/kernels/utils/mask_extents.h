// Where a RetNet mask tensor is zero, its tiles contribute exactly nothing: S = (Q K^T) * 0 adds 0 to the
// normaliser, to O and to every gradient.  The reference streams and multiplies every tile regardless
// (reference csrc/kernels/retnet/smemfuse/smemfuse.h walks all of seq_k for every row block); RetNet's own
// mask is lower-triangular, so half of that work is on zeros.  Here a scan of the mask, one read of
// H * Sq * Sk halves in one kernel, marks the 32 x 32 tiles that hold a non-zero entry and records for every band of
// 32 query rows the range of kv positions with such a tile; the kernels then walk only the tiles inside their bands'
// ranges.  A block that owns kv positions (the column passes of the backward) takes the range of query rows that reach
// them from the tile marks itself: one byte per lane and band of query rows, a ballot and two bit scans.  Results are
// bit-identical to the dense walk.
//
// Workspace layout (ints, then bytes), nbq = Sq / 32, nbk = Sk / 32:
//   row_lo[H][nbq]  first kv position (a multiple of 32) of the first non-zero 32 x 32 tile of the band
//   row_hi[H][nbq]  one past the last kv position of the last non-zero tile; lo >= hi: the band is empty
//   occ[H][nbq][nbk] bytes: 1 where the 32 x 32 tile has a non-zero entry
#pragma once
#include <hip/hip_runtime.h>

#include "cdna4.h"

namespace aat {

constexpr int kMaskBand = 32;

struct MaskExtents {
  const int* row_lo;
  const int* row_hi;
  const unsigned char* occ;
};

inline size_t mask_extent_ints(int H, int Seq_q, int Seq_k) {
  (void)Seq_k;
  return 2 * (size_t)H * (size_t)(Seq_q / kMaskBand);
}
inline size_t mask_extent_bytes(int H, int Seq_q, int Seq_k) {
  const size_t bytes = mask_extent_ints(H, Seq_q, Seq_k) * sizeof(int) +
                       (size_t)H * (size_t)(Seq_q / kMaskBand) * (size_t)(Seq_k / kMaskBand);
  return (bytes + 255) / 256 * 256;
}
__host__ __device__ inline MaskExtents mask_extents_at(const void* workspace, int H, int Seq_q, int Seq_k) {
  (void)Seq_k;
  const int* p = static_cast<const int*>(workspace);
  const size_t nq = (size_t)H * (size_t)(Seq_q / kMaskBand);
  return {p, p + nq, reinterpret_cast<const unsigned char*>(p + 2 * nq)};
}

// kv range [lo, hi) that the query rows [q0, q0 + rows) of head h can see; rows is a multiple of 32.
AAT_DEV void mask_row_range(const MaskExtents& e, int h, int seq_q, int q0, int rows, int& lo, int& hi) {
  const int nbq = seq_q / kMaskBand;
  lo = 0x7fffffff;
  hi = 0;
  for (int b = q0 / kMaskBand; b < (q0 + rows) / kMaskBand; ++b) {
    const int l = e.row_lo[(size_t)h * nbq + b], u = e.row_hi[(size_t)h * nbq + b];
    lo = l < lo ? l : lo;
    hi = u > hi ? u : hi;
  }
}
// query range [lo, hi) that reaches the kv positions [k0, k0 + rows) of head h, from the tile marks: lane i looks at
// the band of query rows i (+ 64, 128, ...) and the wave's ballot gives the first and the last band with a mark.
// Every lane of the wave must call it (wave-uniform control flow); the result is the same in every lane.
AAT_DEV void mask_col_range(const MaskExtents& e, int h, int seq_q, int seq_k, int k0, int rows, int& lo, int& hi) {
  const int nbq = seq_q / kMaskBand, nbk = seq_k / kMaskBand;
  const unsigned char* occ = e.occ + (size_t)h * nbq * nbk;
  const int lane = threadIdx.x & 63;
  int first = -1, last = -1;
  for (int b0 = 0; b0 < nbq; b0 += 64) {
    const int b = b0 + lane;
    bool marked = false;
    if (b < nbq) {
      for (int c = k0 / kMaskBand; c < (k0 + rows) / kMaskBand; ++c) marked |= occ[(size_t)b * nbk + c] != 0;
    }
    const unsigned long long m = __builtin_amdgcn_ballot_w64(marked);
    if (m != 0) {
      if (first < 0) first = b0 + __builtin_ctzll(m);
      last = b0 + 63 - __builtin_clzll(m);
    }
  }
  lo = first < 0 ? 0x7fffffff : first * kMaskBand;
  hi = first < 0 ? 0 : (last + 1) * kMaskBand;
}
// Tiles [j_begin, j_end) of `tile` positions each that cover [lo, hi) (empty range: j_begin == j_end == 0).
AAT_DEV void mask_tile_range(int lo, int hi, int tile, int n_tiles, int& j_begin, int& j_end) {
  if (lo >= hi) {
    j_begin = j_end = 0;
    return;
  }
  j_begin = lo / tile;
  j_end = (hi + tile - 1) / tile;
  j_end = j_end < n_tiles ? j_end : n_tiles;
}

// One block per (band of 32 query rows, head): marks the non-zero 32 x 32 tiles of the band and writes the
// band's kv range.  -0.0 counts as zero (it multiplies to a zero that adds nothing).
constexpr int kMaskScanThreads = 256;
__global__ void __launch_bounds__(kMaskScanThreads)
mask_scan_rows(const half_t* __restrict__ mask, int* __restrict__ row_lo, int* __restrict__ row_hi,
               unsigned char* __restrict__ occ, int seq_q, int seq_k) {
  extern __shared__ int tile_nz[];                  // [seq_k / 32]
  const int nbq = seq_q / kMaskBand, nbk = seq_k / kMaskBand;
  const int band = blockIdx.x, h = blockIdx.y;
  for (int i = threadIdx.x; i < nbk; i += kMaskScanThreads) tile_nz[i] = 0;
  __syncthreads();
  // a thread owns one 16-byte column of the band (8 kv positions) at a time and ORs its 32 rows: the loads of a
  // column are independent, so many are in flight at once
  const uint4* src = reinterpret_cast<const uint4*>(mask + ((size_t)h * seq_q + (size_t)band * kMaskBand) * seq_k);
  const int chunks_per_row = seq_k / 8;             // 4 chunks per tile column
  for (int c = threadIdx.x; c < chunks_per_row; c += kMaskScanThreads) {
    unsigned any = 0;
#pragma unroll 8
    for (int row = 0; row < kMaskBand; ++row) {
      const uint4 x = src[(size_t)row * chunks_per_row + c];
      any |= x.x | x.y | x.z | x.w;
    }
    if (any & 0x7fff7fffu) tile_nz[c >> 2] = 1;
  }
  __syncthreads();
  unsigned char* o = occ + ((size_t)h * nbq + band) * nbk;
  for (int i = threadIdx.x; i < nbk; i += kMaskScanThreads) o[i] = (unsigned char)tile_nz[i];
  if (threadIdx.x == 0) {
    int lo = 0x7fffffff, hi = 0;
    for (int i = 0; i < nbk; ++i)
      if (tile_nz[i]) {
        lo = lo == 0x7fffffff ? i * kMaskBand : lo;
        hi = (i + 1) * kMaskBand;
      }
    row_lo[(size_t)h * nbq + band] = lo;
    row_hi[(size_t)h * nbq + band] = hi;
  }
}

// The row scan keeps one word of LDS per band of 32 kv positions.
inline bool mask_scan_supported(int Seq_q, int Seq_k) {
  return Seq_q % kMaskBand == 0 && Seq_k % kMaskBand == 0 && Seq_k / kMaskBand <= 1024;
}
// Enqueues the scan of mask [H, Seq_q, Seq_k] into `workspace` (mask_extent_bytes() bytes): one kernel.
inline hipError_t scan_mask(const half_t* mask, int H, int Seq_q, int Seq_k, void* workspace, hipStream_t stream) {
  if (!mask_scan_supported(Seq_q, Seq_k)) return hipErrorInvalidValue;
  int* p = static_cast<int*>(workspace);
  const size_t nq = (size_t)H * (size_t)(Seq_q / kMaskBand);
  unsigned char* occ = reinterpret_cast<unsigned char*>(p + 2 * nq);
  const int nbk = Seq_k / kMaskBand;
  mask_scan_rows<<<dim3(Seq_q / kMaskBand, H), dim3(kMaskScanThreads), nbk * sizeof(int), stream>>>(mask, p, p + nq, occ,
                                                                                               Seq_q, Seq_k);
  return hipGetLastError();
}

// How an entry point is told to walk a mask tensor (the `causal` argument of the *_ex entry points).
constexpr int kMaskDense = 0;     // every tile
constexpr int kMaskCausal = 1;    // the caller promises zeros above the diagonal
constexpr int kMaskScan = 2;      // scan the mask into the workspace, then walk the non-zero ranges
constexpr int kMaskScanned = 3;   // the workspace holds the scan of this mask from an earlier call

struct MaskWalk {
  int causal;
  const int* extents;
};
inline bool mask_mode_ok(int mode, const void* workspace, size_t workspace_bytes, int H, int Seq_q, int Seq_k) {
  if (mode == kMaskDense || mode == kMaskCausal) return true;
  if (mode != kMaskScan && mode != kMaskScanned) return false;
  return workspace != nullptr && workspace_bytes >= mask_extent_bytes(H, Seq_q, Seq_k);
}
inline hipError_t prepare_mask_walk(int mode, const half_t* mask, int H, int Seq_q, int Seq_k, void* workspace,
                                    hipStream_t stream, MaskWalk* walk) {
  walk->causal = mode == kMaskCausal ? 1 : 0;
  walk->extents = nullptr;
  if (!mask_scan_supported(Seq_q, Seq_k)) return hipSuccess;      // beyond the scan's reach (S_kv > 32768): every tile, same bits
  if (mode == kMaskScan) {
    const hipError_t e = scan_mask(mask, H, Seq_q, Seq_k, workspace, stream);
    if (e != hipSuccess) return e;
  }
  if (mode == kMaskScan || mode == kMaskScanned) walk->extents = static_cast<const int*>(workspace);
  return hipSuccess;
}

}  // namespace aat
