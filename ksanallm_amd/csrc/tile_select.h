// Internal view of the tile selector shared by the GEMM entry points.
#pragma once
#include <stddef.h>

namespace ksq {

struct SplitKChoice {
  int mt;     // 16-row tiles of x per workgroup
  int nt;     // 16-column tiles per workgroup
  int waves;  // wavefronts per workgroup, each taking every waves-th k-tile
};

SplitKChoice select_splitk(size_t m, size_t n, size_t k);

}  // namespace ksq
