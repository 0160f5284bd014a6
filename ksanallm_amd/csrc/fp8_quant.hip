// Per-token, per-group FP8 (OCP e4m3) activation quantizer; bit-exact against
//   amax = max(1e-10, max|x|),  s = amax / 448,  q = e4m3_rne_satfinite(x / s)      (IEEE fp32 divisions)
// Each lane owns 8 consecutive channels (one 16-byte load, one 8-byte store); a group of `GROUP` channels is
// GROUP/8 adjacent lanes, reduced with cross-lane shuffles, so a wavefront covers 512 contiguous channels.
#include "ksq_common.h"

namespace ksq {
namespace {

__device__ __forceinline__ uint32_t cvt2_e4m3(float a, float b, uint32_t old, bool hi) {
  // v_cvt_pk_fp8_f32 rounds to nearest even; inputs are clamped to +-448 first so the result never leaves the
  // finite range (NaN passes through and encodes as NaN).
  float ca = fminf(fmaxf(a, -448.0f), 448.0f);
  float cb = fminf(fmaxf(b, -448.0f), 448.0f);
  ca = (a != a) ? a : ca;
  cb = (b != b) ? b : cb;
  return hi ? static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, static_cast<int>(old), true))
            : static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, static_cast<int>(old), false));
}

template <typename T, int GROUP, bool COLMAJOR, bool FUSE>
__global__ void __launch_bounds__(256) fp8_group_quant_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ q,
                                                              float* __restrict__ s, uint32_t m, uint32_t k) {
  constexpr int LPG = GROUP / 8;  // lanes per group
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t total = static_cast<size_t>(m) * k / 8;
  const bool live = i < total;
  const size_t e0 = (live ? i : 0) * 8;
  const uint32_t t = static_cast<uint32_t>(e0 / k);
  const uint32_t col = static_cast<uint32_t>(e0 % k);

  float v[8];
  {
    const uint16_t* src = FUSE ? x + static_cast<size_t>(t) * 2 * k + col : x + e0;
    u32x4 raw = *reinterpret_cast<const u32x4*>(src);
    uint16_t h[8] = {static_cast<uint16_t>(raw.x), static_cast<uint16_t>(raw.x >> 16),
                     static_cast<uint16_t>(raw.y), static_cast<uint16_t>(raw.y >> 16),
                     static_cast<uint16_t>(raw.z), static_cast<uint16_t>(raw.z >> 16),
                     static_cast<uint16_t>(raw.w), static_cast<uint16_t>(raw.w >> 16)};
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = T::to_float(h[j]);
    if (FUSE) {
      u32x4 r2 = *reinterpret_cast<const u32x4*>(src + k);
      uint16_t u[8] = {static_cast<uint16_t>(r2.x), static_cast<uint16_t>(r2.x >> 16),
                       static_cast<uint16_t>(r2.y), static_cast<uint16_t>(r2.y >> 16),
                       static_cast<uint16_t>(r2.z), static_cast<uint16_t>(r2.z >> 16),
                       static_cast<uint16_t>(r2.w), static_cast<uint16_t>(r2.w >> 16)};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float g = v[j];
        float act = g / (1.0f + __expf(-g)) * T::to_float(u[j]);
        v[j] = T::to_float(T::from_float(act));  // the reference rounds silu*mul to T before quantizing
      }
    }
  }

  float amax = 1e-10f;
#pragma unroll
  for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
#pragma unroll
  for (int off = LPG / 2; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, LPG));

  const float scale = amax / 448.0f;
  if (!live) return;
  if ((threadIdx.x % LPG) == 0) {
    const uint32_t g = col / GROUP;
    const uint32_t ng = k / GROUP;
    s[COLMAJOR ? static_cast<size_t>(g) * m + t : static_cast<size_t>(t) * ng + g] = scale;
  }
  u32x2 out{0u, 0u};
  out.x = cvt2_e4m3(v[0] / scale, v[1] / scale, out.x, false);
  out.x = cvt2_e4m3(v[2] / scale, v[3] / scale, out.x, true);
  out.y = cvt2_e4m3(v[4] / scale, v[5] / scale, out.y, false);
  out.y = cvt2_e4m3(v[6] / scale, v[7] / scale, out.y, true);
  *reinterpret_cast<u32x2*>(q + e0) = out;
}

template <typename T, int GROUP>
void launch(const void* x, void* q, void* s, uint32_t m, uint32_t k, bool col, bool fuse, hipStream_t st) {
  const size_t total = static_cast<size_t>(m) * k / 8;
  const unsigned blocks = static_cast<unsigned>(div_up(total, 256));
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  uint8_t* qp = static_cast<uint8_t*>(q);
  float* sp = static_cast<float*>(s);
  if (col) {
    if (fuse) fp8_group_quant_kernel<T, GROUP, true, true><<<blocks, 256, 0, st>>>(xp, qp, sp, m, k);
    else fp8_group_quant_kernel<T, GROUP, true, false><<<blocks, 256, 0, st>>>(xp, qp, sp, m, k);
  } else {
    if (fuse) fp8_group_quant_kernel<T, GROUP, false, true><<<blocks, 256, 0, st>>>(xp, qp, sp, m, k);
    else fp8_group_quant_kernel<T, GROUP, false, false><<<blocks, 256, 0, st>>>(xp, qp, sp, m, k);
  }
}

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT int ksq_fp8_group_quant(const void* x, void* q, void* s, size_t m, size_t k, size_t group,
                                   int column_major, int fuse_silu_mul, int dtype, void* stream) {
  const char* fn = "ksq_fp8_group_quant";
  if (!x || !q || !s) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(q) & 7u) || (reinterpret_cast<uintptr_t>(s) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: x must be 16-byte, q 8-byte, s 4-byte aligned", fn);
  if (group != 32 && group != 64 && group != 128)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: group size %zu not in {32,64,128}", fn, group);
  if (k == 0 || k % group != 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k must be a positive multiple of group", fn);
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  if (m == 0) return KSQ_OK;
  if (m > 0x7fffffffull || k > 0x7fffffffull || m * k / 8 / 256 + 1 > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  const uint32_t mm = static_cast<uint32_t>(m), kk = static_cast<uint32_t>(k);
  hipStream_t st = as_stream(stream);
  const bool col = column_major != 0, fuse = fuse_silu_mul != 0;
#define KSQ_Q(TT, G) launch<TT, G>(x, q, s, mm, kk, col, fuse, st)
  if (dtype == KSQ_F16) {
    if (group == 128) KSQ_Q(F16, 128); else if (group == 64) KSQ_Q(F16, 64); else KSQ_Q(F16, 32);
  } else {
    if (group == 128) KSQ_Q(BF16, 128); else if (group == 64) KSQ_Q(BF16, 64); else KSQ_Q(BF16, 32);
  }
#undef KSQ_Q
  return check_launch(fn);
}
