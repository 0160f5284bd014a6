// Internal view of the tile selector shared by the GEMM entry points.
#pragma once
#include <stddef.h>

namespace ksq {

struct SplitKChoice {
  int mt;     // 16-row tiles of x per workgroup
  int nt;     // 16-column tiles per workgroup
  int waves;  // wavefronts per workgroup; wavefront w takes every waves-th k-tile
};

// m rows in one dense GEMM
SplitKChoice select_splitk(size_t m, size_t n, size_t k);
// same rule for a grid of m_blocks row blocks of 16*mt rows each (MoE: one block per aligned expert segment)
SplitKChoice select_splitk_blocks(int mt, size_t m_blocks, size_t n, size_t k);

// true when the MFMA tile kernel (prefill regime) serves the shape: m above the decode range, group 128 and n a
// multiple of its 256-column workgroup tile
bool use_mfma_tile(size_t m, size_t n, size_t k, size_t group);

}  // namespace ksq
