// Shared host/device helpers of libksq_hip (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <type_traits>

#include "ksq.h"

#define KSQ_EXPORT extern "C" __attribute__((visibility("default")))

namespace ksq {

// ---------------------------------------------------------------------------------------------- errors
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// ---------------------------------------------------------------------------------------------- vector types
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

struct F16 {
  static constexpr int kTag = KSQ_F16;
  // 0x6400 | code is the half 1024 + code
  static constexpr uint32_t kMagic2 = 0x64006400u;
  static constexpr float kMagic = 1024.0f;
  typedef f16x8 frag;
  static __device__ __forceinline__ f32x4 mfma(frag a, frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_float(uint16_t b) {
    return static_cast<float>(__builtin_bit_cast(_Float16, b));
  }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
  }
  static constexpr uint32_t kOne2 = 0x3c003c00u;  // (1.0, 1.0)
  static constexpr uint32_t kNegSym2 = 0xe408e408u;  // (-1032, -1032): minus (magic + 8), the offset of a code without zero point
  // low / high 16 bits of a dword as float
  static __device__ __forceinline__ float lo_to_float(uint32_t w) { return to_float(static_cast<uint16_t>(w)); }
  static __device__ __forceinline__ float hi_to_float(uint32_t w) { return to_float(static_cast<uint16_t>(w >> 16)); }
};

struct BF16 {
  static constexpr int kTag = KSQ_BF16;
  // 0x4300 | code is the bfloat16 128 + code
  static constexpr uint32_t kMagic2 = 0x43004300u;
  static constexpr float kMagic = 128.0f;
  typedef bf16x8 frag;
  static __device__ __forceinline__ f32x4 mfma(frag a, frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_float(uint16_t b) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(b) << 16);
  }
  // round-to-nearest-even, NaN kept quiet
  static __device__ __forceinline__ uint16_t from_float(float f) {
    uint32_t x = __builtin_bit_cast(uint32_t, f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return static_cast<uint16_t>(x >> 16);
  }
  static constexpr uint32_t kOne2 = 0x3f803f80u;
  static constexpr uint32_t kNegSym2 = 0xc308c308u;  // (-136, -136)
  static __device__ __forceinline__ float lo_to_float(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
  static __device__ __forceinline__ float hi_to_float(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
};

template <typename T>
__device__ __forceinline__ typename T::frag as_frag(u32x4 v) {
  return __builtin_bit_cast(typename T::frag, v);
}

// Eight int4 codes of one packed dword -> the MFMA operand (k pairs in ascending order), each element holding
// magic + code.  Nibble i and nibble i+4 are the pair (k = 2i, k = 2i+1).
template <typename T>
__device__ __forceinline__ typename T::frag dequant_magic(uint32_t w) {
  u32x4 v;
  v.x = (w & 0x000f000fu) | T::kMagic2;
  v.y = ((w >> 4) & 0x000f000fu) | T::kMagic2;
  v.z = ((w >> 8) & 0x000f000fu) | T::kMagic2;
  v.w = ((w >> 12) & 0x000f000fu) | T::kMagic2;
  return as_frag<T>(v);
}

// silu(g) * u in fp32, the one definition every kernel that applies the activation uses: exp through the hardware's
// base-2 exponential (one multiply in front, no library expansion), 1 + e, an IEEE division and a multiply, with
// contraction switched off.  Two kernels that must agree bit for bit (the MoE GEMM with the activation in its epilogue
// and the stand-alone activation kernel) then execute the same five roundings; with expf, and with the result flowing
// straight into a conversion, the compiler was free to fuse differently from one call site to the next, which showed as
// one last-place difference in half a million outputs.  Accurate to about 2e-6 relative for |g| < 20, far inside one unit of fp16 / bf16.
__device__ __forceinline__ float silu_mul_f32(float g, float u) {
#pragma clang fp contract(off)
  const float t = g * -1.44269504088896340736f;
  const float e = __builtin_amdgcn_exp2f(t);
  const float d = 1.0f + e;
  const float q = g / d;
  float y = q * u;
  // the product exists as an fp32 value of its own: without this the compiler may fold the multiply into the caller's
  // conversion to fp16 (one mixed-precision instruction that rounds once), which differs from rounding twice at ties
  asm("" : "+v"(y));
  return y;
}

__device__ __forceinline__ uint32_t pack2(uint16_t lo, uint16_t hi) {
  return static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
}

inline size_t div_up(size_t a, size_t b) { return (a + b - 1) / b; }
inline size_t round_up(size_t a, size_t b) { return div_up(a, b) * b; }


// A kernel that asks for more dynamic LDS than the default limit needs hipFuncSetAttribute once per device (the
// attribute belongs to the function as loaded on that device; a process that drives several GPUs from several threads
// calls in here from each).  `done` holds one bit per device ordinal, set after the attribute has been accepted.
// Returns 0, or the KSQ_ERR_LAUNCH code after recording the message.
inline int allow_dynamic_lds(std::atomic<uint64_t>& done, const void* kernel, int bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) return fail(KSQ_ERR_LAUNCH, "cannot tell the current device");
  const uint64_t bit = uint64_t(1) << dev;
  if (done.load(std::memory_order_acquire) & bit) return 0;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return fail(KSQ_ERR_LAUNCH, "hipFuncSetAttribute(LDS %d): %s", bytes, hipGetErrorString(e));
  done.fetch_or(bit, std::memory_order_release);
  return 0;
}

// f(integral_constant<N>) for the smallest N in LO..HI with count <= N (N = HI when there is none)
template <int LO, int HI, typename F>
__device__ __forceinline__ void for_tile_count(uint32_t count, F&& f) {
  if constexpr (LO >= HI) {
    f(std::integral_constant<int, HI>{});
  } else {
    if (count <= static_cast<uint32_t>(LO))
      f(std::integral_constant<int, LO>{});
    else
      for_tile_count<LO + 1, HI>(count, f);
  }
}

}  // namespace ksq
