// Second pass of the split-K tile kernels: sums the fp32 partial tiles and rounds to the output type.
#pragma once

#include "ksq_common.h"
#include "tile_work.h"

namespace ksq {

// Partial tiles lie as [slot][part][BM][256] fp32.  One workgroup sums 2048 consecutive elements (8 rows) of one slot,
// 8 per thread, in part order, and writes the rows and columns that are inside the matrix.
// y32 given: the sums are stored as they are, [M, N] fp32, instead of rounded to T (the verification entry points).
template <typename T, int BM>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ partial, uint16_t* __restrict__ y,
                                                            uint32_t M, uint32_t N, uint32_t tiles_m, uint32_t tiles_n,
                                                            uint32_t main_items, uint32_t splits, float* __restrict__ y32 = nullptr) {
  constexpr uint32_t BN = 256;
  constexpr uint32_t kBlocksPerTile = BM * BN / 2048;
  const uint32_t slot = blockIdx.x / kBlocksPerTile;
  const uint32_t e = (blockIdx.x % kBlocksPerTile) * 2048 + threadIdx.x * 8;
  uint32_t tile_m, tile_n;
  tile_of_slot(slot, tiles_m, tiles_n, main_items, &tile_m, &tile_n);
  const uint32_t row = tile_m * BM + e / BN, col = tile_n * BN + e % BN;
  if (row >= M || col >= N) return;
  const float* src = partial + static_cast<size_t>(slot) * splits * (BM * BN) + e;
  f32x4 a = *reinterpret_cast<const f32x4*>(src);
  f32x4 b = *reinterpret_cast<const f32x4*>(src + 4);
  for (uint32_t s = 1; s < splits; ++s) {
    a += *reinterpret_cast<const f32x4*>(src + static_cast<size_t>(s) * (BM * BN));
    b += *reinterpret_cast<const f32x4*>(src + static_cast<size_t>(s) * (BM * BN) + 4);
  }
  if (y32) {
    *reinterpret_cast<f32x4*>(y32 + static_cast<size_t>(row) * N + col) = a;
    *reinterpret_cast<f32x4*>(y32 + static_cast<size_t>(row) * N + col + 4) = b;
    return;
  }
  u32x4 o;
  o.x = pack2(T::from_float(a[0]), T::from_float(a[1]));
  o.y = pack2(T::from_float(a[2]), T::from_float(a[3]));
  o.z = pack2(T::from_float(b[0]), T::from_float(b[1]));
  o.w = pack2(T::from_float(b[2]), T::from_float(b[3]));
  *reinterpret_cast<u32x4*>(y + static_cast<size_t>(row) * N + col) = o;
}

// Second pass of the decode kernel when K is cut over workgroups: y[i] = T(sum over parts of partial[s][i]), parts in
// order, 4 outputs per thread (m*n is a multiple of 16).
template <typename T>
__global__ void __launch_bounds__(256) parts_reduce_kernel(const float* __restrict__ partial, uint16_t* __restrict__ y,
                                                           size_t mn, uint32_t parts, float* __restrict__ y32 = nullptr) {
  const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i >= mn) return;
  f32x4 a = *reinterpret_cast<const f32x4*>(partial + i);
  for (uint32_t s = 1; s < parts; ++s) a += *reinterpret_cast<const f32x4*>(partial + s * mn + i);
  if (y32) {
    *reinterpret_cast<f32x4*>(y32 + i) = a;
    return;
  }
  u32x2 o;
  o.x = pack2(T::from_float(a[0]), T::from_float(a[1]));
  o.y = pack2(T::from_float(a[2]), T::from_float(a[3]));
  *reinterpret_cast<u32x2*>(y + i) = o;
}

}  // namespace ksq
