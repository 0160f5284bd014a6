// Per-token, per-group FP8 (OCP e4m3) activation quantizer; bit-exact against
//   amax = max(1e-10, max|x|),  s = amax / 448,  q = e4m3_rne_satfinite(x / s)      (IEEE fp32 divisions)
// Each lane owns 8 consecutive channels (one 16-byte load, one 8-byte store); a group of `GROUP` channels is
// GROUP/8 adjacent lanes, reduced with cross-lane shuffles, so a wavefront covers 512 contiguous channels.
//
// The kernels are HBM-bound only if the arithmetic stays small: a full IEEE division is about ten instructions, eight
// of them per lane were more than the memory pipeline leaves time for.  x / s is therefore formed from ONE correctly
// rounded reciprocal per lane, y = 1 / s, and a residual correction per element,
//     q0 = x * y,   r = fma(-q0, s, x)  (exact),   q = fma(r, y, q0),
// which is the correctly rounded quotient (Markstein's theorem) as long as r stays in the normal range;
// tests/cpp/exact_div_test.c checks it against the division for every one of the 2^23 mantissas of s and every
// mantissa a 16-bit input can have.  The sign of x is put back afterwards (x = -0 would otherwise come out as +0).
// Scales outside [2^-80, 2^100] take the division itself; inside, r is exact whenever |x / s| >= 2^-20, and a smaller
// quotient that is one unit in the last place off still converts to the same signed zero.
#include <type_traits>

#include "exact_div.h"
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

// two quotients that are known to lie within +-448 * (1 + 2^-23), or NaN: no clamp in front of the conversion
__device__ __forceinline__ uint32_t cvt2_e4m3_in_range(float a, float b, uint32_t old, bool hi) {
  return hi ? static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, static_cast<int>(old), true))
            : static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, static_cast<int>(old), false));
}

// fp32 activations (the reference instantiates its quantizer for float as well): the same kernel with 32-byte loads and
// IEEE divisions throughout - the reciprocal-and-correction form above is proven for inputs of at most 11 significant
// bits, and this type is not on any model's hot path.
struct F32 {
  static constexpr int kTag = KSQ_F32;
};

// eight consecutive channels of one row as floats
template <typename T>
__device__ __forceinline__ void load8(const void* x, size_t e, float (&v)[8]) {
  if constexpr (std::is_same<T, F32>::value) {
    const float* src = static_cast<const float*>(x) + e;
    const f32x4 a = *reinterpret_cast<const f32x4*>(src), b = *reinterpret_cast<const f32x4*>(src + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] = a[j];
      v[4 + j] = b[j];
    }
  } else {
    const u32x4 raw = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(x) + e);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[2 * j] = T::to_float(static_cast<uint16_t>(raw[j] & 0xffffu));
      v[2 * j + 1] = T::to_float(static_cast<uint16_t>(raw[j] >> 16));
    }
  }
}

template <typename T>
__device__ __forceinline__ float load1(const void* x, size_t e) {
  if constexpr (std::is_same<T, F32>::value) return static_cast<const float*>(x)[e];
  else return T::to_float(static_cast<const uint16_t*>(x)[e]);
}

// Grid: x = chunks of BLOCK*8 channels of a row, y and z = the row (token) as z * gridDim.y + y, so that no index needs
// an integer division (about fifty instructions on this ISA, more than the rest of the kernel).  Lanes past the end of
// the row in its last chunk idle; groups never straddle a chunk.
template <typename T, int GROUP, bool COLMAJOR, bool FUSE, int BLOCK>
__global__ void __launch_bounds__(BLOCK) fp8_group_quant_kernel(const void* __restrict__ x, uint8_t* __restrict__ q,
                                                                float* __restrict__ s, uint32_t m, uint32_t k) {
  constexpr bool kF32 = std::is_same<T, F32>::value;
  constexpr int LPG = GROUP / 8;  // lanes per group
  const uint32_t row = blockIdx.z * gridDim.y + blockIdx.y;
  const uint32_t col0 = (blockIdx.x * BLOCK + threadIdx.x) * 8;
  const bool live = row < m && col0 < k;
  const uint32_t t = live ? row : 0;
  const uint32_t col = live ? col0 : 0;
  const size_t e0 = static_cast<size_t>(t) * k + col;

  float v[8];
  {
    const size_t src = FUSE ? static_cast<size_t>(t) * 2 * k + col : e0;
    load8<T>(x, src, v);
    if (FUSE) {
      float u[8];
      load8<T>(x, src + k, u);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // the one definition of silu * mul every kernel here uses (ksq_common.h), so that the int4 and the block-fp8
        // expert paths apply the same activation
        const float act = silu_mul_f32(v[j], u[j]);
        if constexpr (kF32) v[j] = act;
        else v[j] = T::to_float(T::from_float(act));  // the reference rounds silu*mul to T before quantizing
      }
    }
  }

  float amax = 1e-10f;
#pragma unroll
  for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
#pragma unroll
  for (int off = LPG / 2; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, LPG));

  // amax / 448, correctly rounded, by the same reciprocal-and-correction (amax has at most 11 significant bits, or is
  // the floor 1e-10, whose quotient is a constant)
  float scale;
  {
    constexpr float y448 = 1.0f / 448.0f;
    const float q0 = amax * y448;
    const float r = __builtin_fmaf(-q0, 448.0f, amax);
    scale = __builtin_fmaf(r, y448, q0);
    scale = amax == 1e-10f ? 1e-10f / 448.0f : scale;
    scale = (!kF32 && amax >= 0x1p-60f && amax <= 0x1p100f) ? scale : amax / 448.0f;
  }
  if (!live) return;
  if ((threadIdx.x % LPG) == 0) {
    const uint32_t g = col / GROUP;
    const uint32_t ng = k / GROUP;
    s[COLMAJOR ? static_cast<size_t>(g) * m + t : static_cast<size_t>(t) * ng + g] = scale;
  }
  u32x2 out{0u, 0u};
  const ExactDiv div(scale);
  if (!kF32 && div.fast) {
    // every |v| <= amax (an infinite v makes amax, hence the scale, infinite: not this branch), so the quotients stay
    // within 448 * (1 + 2^-23), which the conversion rounds to 448 by itself
    out.x = cvt2_e4m3_in_range(div(v[0]), div(v[1]), out.x, false);
    out.x = cvt2_e4m3_in_range(div(v[2]), div(v[3]), out.x, true);
    out.y = cvt2_e4m3_in_range(div(v[4]), div(v[5]), out.y, false);
    out.y = cvt2_e4m3_in_range(div(v[6]), div(v[7]), out.y, true);
  } else {
    out.x = cvt2_e4m3(v[0] / scale, v[1] / scale, out.x, false);
    out.x = cvt2_e4m3(v[2] / scale, v[3] / scale, out.x, true);
    out.y = cvt2_e4m3(v[4] / scale, v[5] / scale, out.y, false);
    out.y = cvt2_e4m3(v[6] / scale, v[7] / scale, out.y, true);
  }
  *reinterpret_cast<u32x2*>(q + e0) = out;
}

template <typename T, int GROUP, int BLOCK>
void launch_block(const void* x, void* q, void* s, uint32_t m, uint32_t k, bool col, bool fuse, hipStream_t st) {
  const unsigned gy = m < 32768u ? m : 32768u;
  const dim3 grid(static_cast<unsigned>(div_up(k, BLOCK * 8)), gy, static_cast<unsigned>(div_up(m, gy)));
  const void* xp = x;
  uint8_t* qp = static_cast<uint8_t*>(q);
  float* sp = static_cast<float*>(s);
  if (col) {
    if (fuse) fp8_group_quant_kernel<T, GROUP, true, true, BLOCK><<<grid, BLOCK, 0, st>>>(xp, qp, sp, m, k);
    else fp8_group_quant_kernel<T, GROUP, true, false, BLOCK><<<grid, BLOCK, 0, st>>>(xp, qp, sp, m, k);
  } else {
    if (fuse) fp8_group_quant_kernel<T, GROUP, false, true, BLOCK><<<grid, BLOCK, 0, st>>>(xp, qp, sp, m, k);
    else fp8_group_quant_kernel<T, GROUP, false, false, BLOCK><<<grid, BLOCK, 0, st>>>(xp, qp, sp, m, k);
  }
}

template <typename T, int GROUP>
void launch(const void* x, void* q, void* s, uint32_t m, uint32_t k, bool col, bool fuse, hipStream_t st) {
  // workgroup width by row length: a short row would leave most of a wide workgroup idle
  if (k <= 512) launch_block<T, GROUP, 64>(x, q, s, m, k, col, fuse, st);
  else if (k <= 1024) launch_block<T, GROUP, 128>(x, q, s, m, k, col, fuse, st);
  else launch_block<T, GROUP, 256>(x, q, s, m, k, col, fuse, st);
}


// ---- per-channel / per-tensor quantization (one fp32 scale per row of [channels, size]) ------------------------------
constexpr float kMinScale = 1.0f / 448.0f / 512.0f;

__global__ void fp8_scale_clear_kernel(float* __restrict__ scale, uint32_t channels) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i < channels) scale[i] = 0.f;
}

// scale[c] = max(amax(|x[c, :]|) / 448, 1 / (448 * 512)).  Every workgroup folds its maximum in with an integer
// atomic max on the float's bits (all candidates are positive, so the orders agree); scale[] starts at 0.
template <typename T>
__global__ void __launch_bounds__(256) fp8_channel_scale_kernel(const void* __restrict__ x, float* __restrict__ scale,
                                                                size_t size, bool vec) {
  const size_t row = static_cast<size_t>(blockIdx.y) * size;  // first element of this channel
  const size_t tid = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  float amax = 0.f;
  if (vec) {
    auto fold = [&](const float (&v)[8]) {
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
    };
    const size_t n8 = size / 8;
    size_t i = tid;
    // four independent loads in flight per thread: one load per trip leaves the pass waiting on memory latency
    for (; i + 3 * stride < n8; i += 4 * stride) {
      float r0[8], r1[8], r2[8], r3[8];
      load8<T>(x, row + i * 8, r0);
      load8<T>(x, row + (i + stride) * 8, r1);
      load8<T>(x, row + (i + 2 * stride) * 8, r2);
      load8<T>(x, row + (i + 3 * stride) * 8, r3);
      fold(r0);
      fold(r1);
      fold(r2);
      fold(r3);
    }
    for (; i < n8; i += stride) {
      float r0[8];
      load8<T>(x, row + i * 8, r0);
      fold(r0);
    }
  } else {
    for (size_t i = tid; i < size; i += stride) amax = fmaxf(amax, fabsf(load1<T>(x, row + i)));
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
  // one atomic per workgroup: atomics on one address are served one after the other (one per wavefront of a full grid
  // cost more time than reading the tensor)
  __shared__ float wave_max[4];
  if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = amax;
  __syncthreads();
  if (threadIdx.x == 0) {
    amax = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
    const float sc = fmaxf(amax / 448.0f, kMinScale);
    atomicMax(reinterpret_cast<unsigned int*>(scale + blockIdx.y), __float_as_uint(sc));
  }
}

// q[c, i] = e4m3(clamp(x[c, i] / scale[c], -448, 448)), IEEE division, round to nearest even
template <typename T>
__global__ void __launch_bounds__(256) fp8_channel_quant_kernel(const void* __restrict__ x, uint8_t* __restrict__ q,
                                                                const float* __restrict__ scale, size_t size, bool vec) {
  const size_t base = static_cast<size_t>(blockIdx.y) * size;
  const float sc = scale[blockIdx.y];
  const ExactDiv div(sc);
  const size_t tid = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  if (vec) {
    for (size_t i = tid; i < size / 8; i += stride) {
      float v[8];
      load8<T>(x, base + i * 8, v);
      // with a scale handed in by the caller an input may be infinite where the scale is not: such a lane keeps the
      // division (a branch, not a select per element: a select would evaluate the division for every element)
      float mx = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) mx = fmaxf(mx, __builtin_fabsf(v[j]));
      if (std::is_same<T, F32>::value || mx == __builtin_inff()) {  // (fp32 inputs: the division, see F32)
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = v[j] / sc;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = div(v[j]);
      }
      u32x2 out{0u, 0u};
      out.x = cvt2_e4m3(v[0], v[1], out.x, false);
      out.x = cvt2_e4m3(v[2], v[3], out.x, true);
      out.y = cvt2_e4m3(v[4], v[5], out.y, false);
      out.y = cvt2_e4m3(v[6], v[7], out.y, true);
      *reinterpret_cast<u32x2*>(q + base + i * 8) = out;
    }
  } else {
    for (size_t i = tid; i < size; i += stride)
      q[base + i] = static_cast<uint8_t>(cvt2_e4m3(load1<T>(x, base + i) / sc, 0.f, 0u, false) & 0xffu);
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
  if (dtype != KSQ_F16 && dtype != KSQ_BF16 && dtype != KSQ_F32)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16, bf16 or f32", fn);
  if (m == 0) return KSQ_OK;
  if (m > 0x7fffffffull || k > 0x7fffffffull || m * k / 8 / 256 + 1 > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  const uint32_t mm = static_cast<uint32_t>(m), kk = static_cast<uint32_t>(k);
  hipStream_t st = as_stream(stream);
  const bool col = column_major != 0, fuse = fuse_silu_mul != 0;
#define KSQ_Q(TT, G) launch<TT, G>(x, q, s, mm, kk, col, fuse, st)
  if (dtype == KSQ_F32) {
    if (group == 128) KSQ_Q(F32, 128); else if (group == 64) KSQ_Q(F32, 64); else KSQ_Q(F32, 32);
  } else if (dtype == KSQ_F16) {
    if (group == 128) KSQ_Q(F16, 128); else if (group == 64) KSQ_Q(F16, 64); else KSQ_Q(F16, 32);
  } else {
    if (group == 128) KSQ_Q(BF16, 128); else if (group == 64) KSQ_Q(BF16, 64); else KSQ_Q(BF16, 32);
  }
#undef KSQ_Q
  return check_launch(fn);
}

KSQ_EXPORT int ksq_fp8_channel_quant(const void* x, void* q, void* scale, size_t channels, size_t size, int is_static,
                                     int dtype, void* stream) {
  const char* fn = "ksq_fp8_channel_quant";
  if (!x || !q || !scale) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (dtype != KSQ_F16 && dtype != KSQ_BF16 && dtype != KSQ_F32)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16, bf16 or f32", fn);
  if ((reinterpret_cast<uintptr_t>(x) & (dtype == KSQ_F32 ? 3u : 1u)) || (reinterpret_cast<uintptr_t>(scale) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: x must be aligned to its element size, scale to 4 bytes", fn);
  if (channels == 0 || size == 0) return KSQ_OK;
  if (channels > 65535) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: at most 65535 channels", fn);
  // 16-byte loads and 8-byte stores need rows that start on those boundaries
  const bool vec = size % 8 == 0 && aligned16(x) && (reinterpret_cast<uintptr_t>(q) & 7u) == 0;
  const size_t work = vec ? size / 8 : size;
  size_t bx = div_up(work, 256);
  if (bx > 1024) bx = 1024;
  const dim3 grid(static_cast<unsigned>(bx), static_cast<unsigned>(channels), 1);
  hipStream_t st = as_stream(stream);
  const void* xp = x;
  float* sp = static_cast<float*>(scale);
  if (!is_static) {
    fp8_scale_clear_kernel<<<static_cast<unsigned>(div_up(channels, 256)), 256, 0, st>>>(sp, static_cast<uint32_t>(channels));
    // two workgroups per CU read as fast as more do and keep the atomics few
    const dim3 sgrid(static_cast<unsigned>(bx < 512 ? bx : 512), static_cast<unsigned>(channels), 1);
    if (dtype == KSQ_F32) fp8_channel_scale_kernel<F32><<<sgrid, 256, 0, st>>>(xp, sp, size, vec);
    else if (dtype == KSQ_F16) fp8_channel_scale_kernel<F16><<<sgrid, 256, 0, st>>>(xp, sp, size, vec);
    else fp8_channel_scale_kernel<BF16><<<sgrid, 256, 0, st>>>(xp, sp, size, vec);
  }
  if (dtype == KSQ_F32) fp8_channel_quant_kernel<F32><<<grid, 256, 0, st>>>(xp, static_cast<uint8_t*>(q), sp, size, vec);
  else if (dtype == KSQ_F16) fp8_channel_quant_kernel<F16><<<grid, 256, 0, st>>>(xp, static_cast<uint8_t*>(q), sp, size, vec);
  else fp8_channel_quant_kernel<BF16><<<grid, 256, 0, st>>>(xp, static_cast<uint8_t*>(q), sp, size, vec);
  return check_launch(fn);
}
