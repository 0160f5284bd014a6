// Internal view of the tile selector shared by the GEMM entry points.
#pragma once
#include <stddef.h>

namespace ksq {

struct SplitKChoice {
  int mt;     // 16-row tiles of x per workgroup
  int nt;     // 16-column tiles per workgroup
  int waves;  // wavefronts per workgroup; wavefront w takes every waves-th k-tile
  int parts;  // workgroups along K (1: the whole of K in one workgroup); > 1 needs parts*m*n fp32 of workspace
  int xc;     // 0: x fragments through registers; > 0: x staged through LDS in chunks of xc k-tiles (w4a16_splitk.h)
};

// m rows in one dense GEMM
SplitKChoice select_splitk(size_t m, size_t n, size_t k);
// same rule for a grid of m_blocks row blocks of 16*mt rows each (MoE: one block per aligned expert segment)
SplitKChoice select_splitk_blocks(int mt, size_t m_blocks, size_t n, size_t k);

// The decode-form kernels also serve small problems of more than 32 rows, in blocks of 32 rows; never more than this
// many rows (the workspace queries walk every m up to it).
constexpr size_t kRowBlockMaxM = 512;

// true when the MFMA tile kernel (prefill regime) serves the shape: m above the decode range, a group size the tile
// kernel is built for, and a problem past the size up to which the decode kernel over row blocks is faster
bool use_mfma_tile(size_t m, size_t n, size_t k, size_t group);
// the size rule alone (whatever ksq_set_small_problem_rule says): what the workspace queries size the decode form for
bool small_w4a16_problem(size_t m, size_t n, size_t k, size_t group);

// Grid of the MFMA tile kernel: block_m x 256 output tiles; the first main_items tiles (in the order of tile_work.h)
// are computed whole, the others in `splits` parts of kt_per_split k-steps whose fp32 partial tiles go through the
// workspace.  main_items == 0 and splits > 1: every tile is cut (grids far smaller than the chip).
struct TilePlan {
  int block_m;  // 128 or 256
  unsigned tiles_m, tiles_n, main_items, splits, kt_per_split, grid;
  size_t workspace_bytes;
};
TilePlan plan_mfma_tile(size_t m, size_t n, size_t k);

// Blockwise FP8: whether the MFMA tile kernel replaces the split-K wavefront kernel (above 32 tokens, but for small problems),
// and its grid (block_m is always 256; kt_per_split counts 128-deep k-blocks).
bool use_fp8_tile(size_t m, size_t n, size_t k);
TilePlan plan_fp8_tile(size_t m, size_t n, size_t k);
// W4A8 (w4a8_tile.h): the same regime rule with its own size limit, the same tile shapes with its own costs of a cut along K
bool use_w4a8_tile(size_t m, size_t n, size_t k);
TilePlan plan_w4a8_tile(size_t m, size_t n, size_t k);
// W4A8 streaming kernel (up to 32 tokens): column tiles per workgroup and wavefronts that split K (parts is always 1)
SplitKChoice select_w4a8_splitk(size_t m, size_t n);

}  // namespace ksq
