// Second pass of the split-K tile kernels: sums the fp32 partial tiles and rounds to the output type.
#pragma once

#include "ksq_common.h"

namespace ksq {

// y[m, n] = T(sum over splits of partial[s, m, n]), 8 outputs per thread, summed in split order
template <typename T>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ partial, uint16_t* __restrict__ y,
                                                            size_t mn, uint32_t splits) {
  const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
  if (i >= mn) return;
  f32x4 a = *reinterpret_cast<const f32x4*>(partial + i);
  f32x4 b = *reinterpret_cast<const f32x4*>(partial + i + 4);
  for (uint32_t s = 1; s < splits; ++s) {
    a += *reinterpret_cast<const f32x4*>(partial + s * mn + i);
    b += *reinterpret_cast<const f32x4*>(partial + s * mn + i + 4);
  }
  u32x4 o;
  o.x = pack2(T::from_float(a[0]), T::from_float(a[1]));
  o.y = pack2(T::from_float(a[2]), T::from_float(a[3]));
  o.z = pack2(T::from_float(b[0]), T::from_float(b[1]));
  o.w = pack2(T::from_float(b[2]), T::from_float(b[3]));
  *reinterpret_cast<u32x4*>(y + i) = o;
}

}  // namespace ksq
