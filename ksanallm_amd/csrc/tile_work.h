// Work order of the MFMA tile kernels: which output tile and which part of K a workgroup computes.
//
// A launch holds `main_items` whole tiles (all of K, stored straight to the output) followed by the remaining tiles cut
// into `splits` parts of K each (fp32 partial tiles in the workspace, summed by splitk_reduce_kernel).  main_items == 0
// is the plain split-K launch for grids far smaller than the chip; main_items > 0 is for grids of a few rounds: the
// tiles that would form a last, mostly empty round are cut so finely that they fill the chip once more for a short time.
//
// Workgroup b runs on XCD b%8 and the b/8-th of that XCD's workgroups start in order, 32 at a time (one per CU).  Every
// XCD gets a contiguous range of a linear tile order in which 32 consecutive items form a block of 4 row tiles x 8
// columns (a column = a column tile, or a (column tile, k part) pair in the plain split-K launch): the workgroups that
// share an L2 at any moment read 4 activation tiles and 8 weight strips between them instead of 16 and 2.
#pragma once

#include <stdint.h>

namespace ksq {

struct TileWork {
  uint32_t tile_m, tile_n;
  uint32_t part;        // which part of K
  uint32_t slot;        // index of this tile's partial tiles in the workspace (tiles that are cut only)
  bool direct;          // all of K: store to the output
};

__host__ __device__ __forceinline__ void tile_order(uint32_t lin, uint32_t tiles_m, uint32_t cols, uint32_t* tile_m, uint32_t* col) {
  constexpr uint32_t GN = 8;
  const uint32_t band_items = tiles_m * GN;
  const uint32_t band = lin / band_items;
  const uint32_t c0 = band * GN;
  const uint32_t width = (cols - c0) < GN ? (cols - c0) : GN;
  const uint32_t within = lin - band * band_items;
  *tile_m = within / width;
  *col = c0 + within % width;
}

__host__ __device__ __forceinline__ uint32_t xcd_range(uint32_t b, uint32_t total) {
  const uint32_t per = total / 8, rem = total % 8;
  const uint32_t xcd = b % 8, local = b / 8;
  return xcd * per + (xcd < rem ? xcd : rem) + local;  // XCDs 0..rem-1 own per+1 items
}

// The grouped (MoE) launches size their grid for the largest number of row blocks an alignment can produce, and the
// blocks past the aligned length - up to half of the grid, all at the end of each band of the linear order - leave at
// once.  A contiguous range per XCD would hand some XCDs nothing but such blocks; here every run of 256 consecutive
// workgroups covers 256 consecutive items, 32 consecutive ones (4 row blocks x 8 column tiles) per XCD, so the blocks
// that compute are spread over all XCDs at every moment of the launch.
__host__ __device__ __forceinline__ uint32_t xcd_interleave(uint32_t b, uint32_t total) {
  if (b >= total / 256 * 256) return b;
  return (b & ~255u) + (b % 8) * 32 + (b % 256) / 8;
}

__host__ __device__ __forceinline__ TileWork tile_work(uint32_t b, uint32_t tiles_m, uint32_t tiles_n, uint32_t main_items,
                                              uint32_t splits, bool grouped = false) {
  TileWork w;
  if (grouped) {
    tile_order(xcd_interleave(b, tiles_m * tiles_n), tiles_m, tiles_n, &w.tile_m, &w.tile_n);
    w.part = 0;
    w.slot = 0;
    w.direct = true;
  } else if (main_items == 0) {
    const uint32_t cols = tiles_n * splits;
    uint32_t col;
    tile_order(xcd_range(b, tiles_m * cols), tiles_m, cols, &w.tile_m, &col);
    w.part = col % splits;
    w.tile_n = col / splits;
    w.slot = w.tile_m * tiles_n + w.tile_n;
    w.direct = splits == 1;
  } else if (b < main_items) {
    tile_order(xcd_range(b, main_items), tiles_m, tiles_n, &w.tile_m, &w.tile_n);
    w.part = 0;
    w.slot = 0;
    w.direct = true;
  } else {
    const uint32_t t = b - main_items;
    w.slot = t / splits;
    w.part = t % splits;
    tile_order(main_items + w.slot, tiles_m, tiles_n, &w.tile_m, &w.tile_n);
    w.direct = false;
  }
  return w;
}

// tile of workspace slot `slot` (the inverse of the above for the reduction pass)
__host__ __device__ __forceinline__ void tile_of_slot(uint32_t slot, uint32_t tiles_m, uint32_t tiles_n, uint32_t main_items,
                                             uint32_t* tile_m, uint32_t* tile_n) {
  if (main_items == 0) {
    *tile_m = slot / tiles_n;
    *tile_n = slot % tiles_n;
  } else {
    tile_order(main_items + slot, tiles_m, tiles_n, tile_m, tile_n);
  }
}

}  // namespace ksq
