// Host check of the tile kernels' work order (ksanallm_amd/csrc/tile_work.h): over a launch every (tile, part of K)
// pair is taken by exactly one workgroup, whole tiles and cut tiles do not overlap, and tile_of_slot inverts the slot
// numbering.  Built with g++ (the header's __host__ __device__ markers are defined away on the command line).
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "tile_work.h"

using namespace ksq;

static int check(uint32_t tiles_m, uint32_t tiles_n, uint32_t main_items, uint32_t splits) {
  const uint32_t tiles = tiles_m * tiles_n;
  const uint32_t grid = main_items + (tiles - main_items) * splits;
  std::vector<int> seen(static_cast<size_t>(tiles) * splits, 0);
  std::vector<int> whole(tiles, 0);
  for (uint32_t b = 0; b < grid; ++b) {
    const TileWork w = tile_work(b, tiles_m, tiles_n, main_items, splits);
    if (w.tile_m >= tiles_m || w.tile_n >= tiles_n || w.part >= splits) return 1;
    const uint32_t t = w.tile_m * tiles_n + w.tile_n;
    if (w.direct) {
      if (whole[t]++) return 2;
    } else {
      if (seen[static_cast<size_t>(t) * splits + w.part]++) return 3;
      uint32_t tm, tn;
      tile_of_slot(w.slot, tiles_m, tiles_n, main_items, &tm, &tn);
      if (tm != w.tile_m || tn != w.tile_n) return 4;
      if (w.slot >= tiles - main_items) return 5;
    }
  }
  for (uint32_t t = 0; t < tiles; ++t) {
    int parts = 0;
    for (uint32_t s = 0; s < splits; ++s) parts += seen[static_cast<size_t>(t) * splits + s];
    const bool ok = (whole[t] == 1 && parts == 0) || (whole[t] == 0 && parts == static_cast<int>(splits));
    if (!ok) return 6;
  }
  return 0;
}

// grouped launches: every tile once, all direct; any 256 consecutive workgroups that lie inside the interleaved part
// take 256 consecutive items, the 32 of one XCD (b % 8) consecutive among them
static int check_grouped(uint32_t tiles_m, uint32_t tiles_n) {
  const uint32_t tiles = tiles_m * tiles_n;
  std::vector<int> whole(tiles, 0);
  for (uint32_t b = 0; b < tiles; ++b) {
    const TileWork w = tile_work(b, tiles_m, tiles_n, 0, 1, true);
    if (w.tile_m >= tiles_m || w.tile_n >= tiles_n || !w.direct || w.part != 0) return 1;
    if (whole[w.tile_m * tiles_n + w.tile_n]++) return 2;
    const uint32_t lin = xcd_interleave(b, tiles);
    if (lin >= tiles) return 3;
    if (b < tiles / 256 * 256) {
      if (lin / 256 != b / 256) return 4;
      if ((lin % 256) / 32 != b % 8) return 5;
    } else if (lin != b) {
      return 6;
    }
  }
  return 0;
}

int main() {
  int cases = 0;
  for (uint32_t tm : {1u, 3u, 16u, 33u, 510u, 766u})
    for (uint32_t tn : {1u, 7u, 16u, 28u}) {
      const int rc = check_grouped(tm, tn);
      ++cases;
      if (rc) {
        std::printf("FAIL grouped rc=%d tiles_m=%u tiles_n=%u\n", rc, tm, tn);
        return 1;
      }
    }
  const uint32_t ms[] = {1, 2, 3, 5, 16, 33};
  const uint32_t ns[] = {1, 7, 8, 9, 20, 53, 100};
  for (uint32_t tm : ms)
    for (uint32_t tn : ns)
      for (uint32_t splits : {1u, 2u, 3u, 8u, 16u}) {
        const uint32_t tiles = tm * tn;
        for (uint32_t main_items : {0u, tiles / 256 * 256, tiles > 3 ? tiles - 3 : 0u}) {
          if (main_items > tiles) continue;
          const int rc = check(tm, tn, main_items, splits);
          ++cases;
          if (rc) {
            std::printf("FAIL rc=%d tiles_m=%u tiles_n=%u main=%u splits=%u\n", rc, tm, tn, main_items, splits);
            return 1;
          }
        }
      }
  std::printf("OK %d cases\n", cases);
  return 0;
}
