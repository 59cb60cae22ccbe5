// Where a RetNet mask tensor is zero, its tiles contribute exactly nothing: S = (Q K^T) * 0 adds 0 to the
// normaliser, to O and to every gradient.  The reference streams and multiplies every tile regardless
// (reference csrc/kernels/retnet/smemfuse/smemfuse.h walks all of seq_k for every row block); RetNet's own
// mask is lower-triangular, so half of that work is on zeros.  Here a scan of the mask, one read of
// H * Sq * Sk halves, records for every band of 32 query rows the range of kv positions that hold a
// non-zero entry and for every band of 32 kv positions the range of query rows; the kernels then walk
// only the tiles inside their bands' ranges.  Results are bit-identical to the dense walk.
//
// Workspace layout (ints, then bytes), nbq = Sq / 32, nbk = Sk / 32:
//   row_lo[H][nbq]  first kv position (a multiple of 32) of the first non-zero 32 x 32 tile of the band
//   row_hi[H][nbq]  one past the last kv position of the last non-zero tile; lo >= hi: the band is empty
//   col_lo[H][nbk]  the same for a band of kv positions, in query positions
//   col_hi[H][nbk]
//   occ[H][nbq][nbk] bytes: 1 where the 32 x 32 tile has a non-zero entry (scratch of the scan)
#pragma once
#include <hip/hip_runtime.h>

#include "cdna4.h"

namespace aat {

constexpr int kMaskBand = 32;

struct MaskExtents {
  const int* row_lo;
  const int* row_hi;
  const int* col_lo;
  const int* col_hi;
};

inline size_t mask_extent_ints(int H, int Seq_q, int Seq_k) {
  return 2 * (size_t)H * (size_t)(Seq_q / kMaskBand) + 2 * (size_t)H * (size_t)(Seq_k / kMaskBand);
}
inline size_t mask_extent_bytes(int H, int Seq_q, int Seq_k) {
  const size_t bytes = mask_extent_ints(H, Seq_q, Seq_k) * sizeof(int) +
                       (size_t)H * (size_t)(Seq_q / kMaskBand) * (size_t)(Seq_k / kMaskBand);
  return (bytes + 255) / 256 * 256;
}
__host__ __device__ inline MaskExtents mask_extents_at(const void* workspace, int H, int Seq_q, int Seq_k) {
  const int* p = static_cast<const int*>(workspace);
  const size_t nq = (size_t)H * (size_t)(Seq_q / kMaskBand), nk = (size_t)H * (size_t)(Seq_k / kMaskBand);
  return {p, p + nq, p + 2 * nq, p + 2 * nq + nk};
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
// query range [lo, hi) that reaches the kv positions [k0, k0 + rows) of head h.
AAT_DEV void mask_col_range(const MaskExtents& e, int h, int seq_k, int k0, int rows, int& lo, int& hi) {
  const int nbk = seq_k / kMaskBand;
  lo = 0x7fffffff;
  hi = 0;
  for (int b = k0 / kMaskBand; b < (k0 + rows) / kMaskBand; ++b) {
    const int l = e.col_lo[(size_t)h * nbk + b], u = e.col_hi[(size_t)h * nbk + b];
    lo = l < lo ? l : lo;
    hi = u > hi ? u : hi;
  }
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

// One block per head: the query range of every band of 32 kv positions, from the tile marks.  The marks
// go through LDS a slab of bands at a time (read along rows, as they lie in memory; scanned along columns).
constexpr int kMaskColSlab = 16 * 1024;             // bytes of tile marks held in LDS at a time
__global__ void __launch_bounds__(kMaskScanThreads)
mask_scan_cols(const unsigned char* __restrict__ occ, int* __restrict__ col_lo, int* __restrict__ col_hi, int seq_q,
               int seq_k) {
  __shared__ unsigned char slab[kMaskColSlab];
  const int nbq = seq_q / kMaskBand, nbk = seq_k / kMaskBand;
  const int h = blockIdx.x;
  const unsigned char* src = occ + (size_t)h * nbq * nbk;
  const int bands_per_slab = kMaskColSlab / nbk < 1 ? 1 : kMaskColSlab / nbk;
  // a thread owns the columns cb, cb + 256, ...; at most 4 of them for seq_k <= 32768 (checked by the launcher)
  int lo[4], hi[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    lo[i] = 0x7fffffff;
    hi[i] = 0;
  }
  for (int b0 = 0; b0 < nbq; b0 += bands_per_slab) {
    const int nb = nbq - b0 < bands_per_slab ? nbq - b0 : bands_per_slab;
    __syncthreads();
    for (int i = threadIdx.x; i < nb * nbk; i += kMaskScanThreads) slab[i] = src[(size_t)b0 * nbk + i];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int cb = threadIdx.x + i * kMaskScanThreads;
      if (cb < nbk) {
#pragma unroll 8
        for (int b = 0; b < nb; ++b) {              // selects, no branches: the LDS reads of a column overlap
          const bool nz = slab[b * nbk + cb] != 0;
          lo[i] = (nz && lo[i] == 0x7fffffff) ? (b0 + b) * kMaskBand : lo[i];
          hi[i] = nz ? (b0 + b + 1) * kMaskBand : hi[i];
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int cb = threadIdx.x + i * kMaskScanThreads;
    if (cb < nbk) {
      col_lo[(size_t)h * nbk + cb] = lo[i];
      col_hi[(size_t)h * nbk + cb] = hi[i];
    }
  }
}

// The column scan keeps one running range per thread for up to four bands of 32 kv positions.
inline bool mask_scan_supported(int Seq_q, int Seq_k) {
  return Seq_q % kMaskBand == 0 && Seq_k % kMaskBand == 0 && Seq_k / kMaskBand <= 4 * kMaskScanThreads &&
         Seq_k / kMaskBand <= kMaskColSlab;
}
// Enqueues the scan of mask [H, Seq_q, Seq_k] into `workspace` (mask_extent_bytes() bytes).
inline hipError_t scan_mask(const half_t* mask, int H, int Seq_q, int Seq_k, void* workspace, hipStream_t stream) {
  if (!mask_scan_supported(Seq_q, Seq_k)) return hipErrorInvalidValue;
  int* p = static_cast<int*>(workspace);
  const size_t nq = (size_t)H * (size_t)(Seq_q / kMaskBand), nk = (size_t)H * (size_t)(Seq_k / kMaskBand);
  unsigned char* occ = reinterpret_cast<unsigned char*>(p + 2 * nq + 2 * nk);
  const int nbk = Seq_k / kMaskBand;
  mask_scan_rows<<<dim3(Seq_q / kMaskBand, H), dim3(kMaskScanThreads), nbk * sizeof(int), stream>>>(mask, p, p + nq, occ,
                                                                                               Seq_q, Seq_k);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  mask_scan_cols<<<dim3(H), dim3(kMaskScanThreads), 0, stream>>>(occ, p + 2 * nq, p + 2 * nq + nk, Seq_q, Seq_k);
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
