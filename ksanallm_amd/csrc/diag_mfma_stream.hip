// ksq_diag_mfma_stream: a stream of independent MFMAs on operands that stay in registers - no memory traffic, no LDS,
// no other arithmetic.  What it sustains is what the matrix pipes deliver under the part's power limit: on operands
// whose bits differ from lane to lane and register to register the clock settles lower than on operands that are all
// the same value, by the same mechanism that bounds the GEMM kernels.  bench.py --mfma-stream times it.
#include "ksq_common.h"

namespace ksq {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ uint32_t mix(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

// 16-bit floats: random sign and mantissa under the exponent of 1.0 (fp16) - finite in both types.
// e4m3 bytes: random but for bit 3, which keeps every byte off the NaN encoding.
template <bool FP8>
__device__ __forceinline__ uint32_t operand_word(uint32_t seed, bool constant) {
  if (constant) return FP8 ? 0x38383838u : 0x3c003c00u;
  const uint32_t h = mix(seed);
  return FP8 ? (h & 0xf7f7f7f7u) : ((h & 0x83ff83ffu) | 0x3c003c00u);
}

// KIND 0 / 1: v_mfma_f32_16x16x32_f16 / _bf16, 32 per iteration as the tile kernels issue them (16 x 2 accumulators).
// KIND 3 / 4: v_mfma_f32_32x32x16_f16 / _bf16, 16 per iteration (8 accumulators x 2 k halves): the same flops.
template <int KIND>
__global__ void __launch_bounds__(512, 1) mfma_stream_16bit(float* sink, int iters, int constant) {
  const uint32_t tid = blockIdx.x * 512 + threadIdx.x;
  u32x4 a[16], b[2];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) a[i][e] = operand_word<false>((tid * 32 + i) * 4 + e, constant);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) b[i][e] = operand_word<false>((tid * 32 + 16 + i) * 4 + e, constant);
  float sum = 0.f;
  if constexpr (KIND == 0 || KIND == 1) {
    f32x4 acc[2][16];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int t = 0; t < 2; ++t)
          acc[t][i] = KIND == 0 ? F16::mfma(as_frag<F16>(b[t]), as_frag<F16>(a[i]), acc[t][i])
                                : BF16::mfma(as_frag<BF16>(b[t]), as_frag<BF16>(a[i]), acc[t][i]);
      a[0].x ^= (it & 1);  // the loop is not invariant
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) sum += acc[t][i][0] + acc[t][i][1] + acc[t][i][2] + acc[t][i][3];
  } else {
    f32x16 acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          acc[i] = KIND == 3 ? __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b[h]),
                                                                     __builtin_bit_cast(f16x8, a[2 * i + h]), acc[i], 0, 0, 0)
                             : __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag<BF16>(b[h]), as_frag<BF16>(a[2 * i + h]), acc[i], 0, 0, 0);
      a[0].x ^= (it & 1);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) sum += acc[i][e];
  }
  if (sum == 12345.678f) sink[tid] = sum;  // never true for these operands; keeps the sums alive
}

// KIND 2: v_mfma_scale_f32_16x16x128_f8f6f4 on e4m3 bytes, 16 per iteration (8 x 2 accumulators);
// KIND 5: v_mfma_scale_f32_32x32x64_f8f6f4, 8 per iteration (4 accumulators x 2 k halves): the same flops.
template <int KIND>
__global__ void __launch_bounds__(512, 1) mfma_stream_fp8(float* sink, int iters, int constant) {
  const uint32_t tid = blockIdx.x * 512 + threadIdx.x;
  i32x8 a[8], b[2];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) a[i][e] = static_cast<int>(operand_word<true>((tid * 16 + i) * 8 + e, constant));
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) b[i][e] = static_cast<int>(operand_word<true>((tid * 16 + 8 + i) * 8 + e, constant));
  float sum = 0.f;
  if constexpr (KIND == 2) {
    f32x4 acc[2][8];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int t = 0; t < 2; ++t)
          acc[t][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[t], a[i], acc[t][i], 0, 0, 0, 0, 0, 0);
      a[0][0] ^= (it & 1);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 8; ++i) sum += acc[t][i][0] + acc[t][i][1] + acc[t][i][2] + acc[t][i][3];
  } else {
    f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[h], a[2 * i + h], acc[i], 0, 0, 0, 0, 0, 0);
      a[0][0] ^= (it & 1);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) sum += acc[i][e];
  }
  if (sum == 12345.678f) sink[tid] = sum;
}

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT double ksq_diag_mfma_stream_flops(int kind, int iters) {
  if (kind < 0 || kind > 5 || iters <= 0) return 0.0;
  // 256 workgroups of 8 wavefronts; per wavefront and iteration 2^19 flops (16-bit forms) or 2^20 (fp8 forms)
  return 256.0 * 8.0 * iters * ((kind == 2 || kind == 5) ? 1048576.0 : 524288.0);
}

KSQ_EXPORT int ksq_diag_mfma_stream(int kind, int constant_operands, int iters, void* sink, void* stream) {
  const char* fn = "ksq_diag_mfma_stream";
  if (kind < 0 || kind > 5) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: kind %d not in 0..5", fn, kind);
  if (iters <= 0 || iters > (1 << 20)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: iters must be in 1..2^20", fn);
  if (!sink) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: sink must hold 256 * 512 floats", fn);
  float* s = static_cast<float*>(sink);
  hipStream_t st = as_stream(stream);
  switch (kind) {
    case 0: mfma_stream_16bit<0><<<256, 512, 0, st>>>(s, iters, constant_operands); break;
    case 1: mfma_stream_16bit<1><<<256, 512, 0, st>>>(s, iters, constant_operands); break;
    case 2: mfma_stream_fp8<2><<<256, 512, 0, st>>>(s, iters, constant_operands); break;
    case 3: mfma_stream_16bit<3><<<256, 512, 0, st>>>(s, iters, constant_operands); break;
    case 4: mfma_stream_16bit<4><<<256, 512, 0, st>>>(s, iters, constant_operands); break;
    default: mfma_stream_fp8<5><<<256, 512, 0, st>>>(s, iters, constant_operands); break;
  }
  return check_launch(fn);
}
