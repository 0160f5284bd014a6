// Prefill-regime W4A16 kernel (MFMA-bound): a workgroup of 8 wavefronts computes a BM x 256 output tile.
//
//   - x (activations) is staged through LDS in MFMA fragment order, double buffered, 64 k per stage: each 1 KiB
//     fragment (16 rows x 32 k) is read back with one conflict-free ds_read_b128 per lane;
//   - packed int4 weights never touch LDS: the wavefronts split the 256 columns between them (WN column tiles of
//     16 each), so every weight fragment belongs to exactly one wavefront, which loads its 1 KiB tiles straight
//     from global memory (16 bytes per lane, one k-tile of 128 every other stage) and dequantizes them in
//     registers to T with scale and zero point applied, (code - zp) * s;
//   - the weights are the row operand of v_mfma_f32_16x16x32 and x the column operand, so a lane ends up with four
//     consecutive output columns of one row and stores them as one 8-byte word; accumulation runs over the whole K
//     inside the MFMA, there is no per-group epilogue.
//
// Workgroup ids are remapped so that the eight XCDs each work on a contiguous band of column tiles and sweep the
// row tiles fastest: the weight band of a workgroup is shared by its neighbours on the same L2.
#pragma once

#include "ksq_common.h"

namespace ksq {

struct TileParams {
  void* y;
  const void* x;
  const void* w;
  const void* scales;
  const void* zeros;
  uint32_t M, N, K;
  uint32_t tiles_m, tiles_n;
};

// dequantize one packed dword (8 codes) to 8 T values with (code - zp) * s applied
template <typename T, bool HAS_ZP>
struct Dequant;

// fp16: 0x6400 | code is the half 1024 + code, and a nibble left in bits 4..7 gives 1024 + 16*code, which saves the
// shifts of the odd nibbles.  code - zp is formed exactly ((1024+code) - (1024+zp), or (1024+16 code)/16 - (64+zp)),
// then multiplied by the scale: one rounding per weight.
template <bool HAS_ZP>
struct Dequant<F16, HAS_ZP> {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  h2 s2, c1, c16;  // (s,s), 1024+zp, 64+zp : the zero point is removed exactly in integers before the scale
  __device__ __forceinline__ void set(uint32_t scale_bits, uint32_t zp) {
    const _Float16 s = __builtin_bit_cast(_Float16, static_cast<uint16_t>(scale_bits));
    const float z = HAS_ZP ? static_cast<float>(zp) : 8.0f;
    s2 = h2{s, s};
    const _Float16 a = static_cast<_Float16>(1024.0f + z), b = static_cast<_Float16>(64.0f + z);
    c1 = h2{a, a};
    c16 = h2{b, b};
  }
  __device__ __forceinline__ F16::frag operator()(uint32_t w) const {
    const h2 sixteenth{static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
    const uint32_t lo0 = (w & 0x000f000fu) | 0x64006400u;   // k = 0,1 : 1024 + code
    const uint32_t hi0 = (w & 0x00f000f0u) | 0x64006400u;   // k = 2,3 : 1024 + 16*code
    const uint32_t w8 = w >> 8;
    const uint32_t lo1 = (w8 & 0x000f000fu) | 0x64006400u;  // k = 4,5
    const uint32_t hi1 = (w8 & 0x00f000f0u) | 0x64006400u;  // k = 6,7
    h2 r0 = (__builtin_bit_cast(h2, lo0) - c1) * s2;
    h2 r1 = (__builtin_bit_cast(h2, hi0) * sixteenth - c16) * s2;
    h2 r2 = (__builtin_bit_cast(h2, lo1) - c1) * s2;
    h2 r3 = (__builtin_bit_cast(h2, hi1) * sixteenth - c16) * s2;
    u32x4 v{__builtin_bit_cast(uint32_t, r0), __builtin_bit_cast(uint32_t, r1), __builtin_bit_cast(uint32_t, r2),
            __builtin_bit_cast(uint32_t, r3)};
    return as_frag<F16>(v);
  }
};

// bf16 has no packed arithmetic on this ISA: codes go through fp32 (byte -> float, one fma each) and are packed
// back with v_cvt_pk_bf16_f32.
template <bool HAS_ZP>
struct Dequant<BF16, HAS_ZP> {
  float s, b;  // s and -zp*s
  __device__ __forceinline__ void set(uint32_t scale_bits, uint32_t zp) {
    s = BF16::lo_to_float(scale_bits);
    b = -(HAS_ZP ? static_cast<float>(zp) : 8.0f) * s;
  }
  static __device__ __forceinline__ uint32_t pk(float a, float c) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    b2 r = __builtin_convertvector(f2{a, c}, b2);
    return __builtin_bit_cast(uint32_t, r);
  }
  __device__ __forceinline__ BF16::frag operator()(uint32_t w) const {
    const uint32_t e = w & 0x0f0f0f0fu;         // nibbles 0,2,4,6 -> k = 0, 4, 1, 5   (nibble i <-> k pair order)
    const uint32_t o = (w >> 4) & 0x0f0f0f0fu;  // nibbles 1,3,5,7 -> k = 2, 6, 3, 7
    // nibble p holds k = {0,2,4,6,1,3,5,7}[p]: even nibbles p=0,2,4,6 -> k=0,4,1,5 ; odd p=1,3,5,7 -> k=2,6,3,7
    const float k0 = static_cast<float>(e & 0xffu), k4 = static_cast<float>((e >> 8) & 0xffu);
    const float k1 = static_cast<float>((e >> 16) & 0xffu), k5 = static_cast<float>(e >> 24);
    const float k2 = static_cast<float>(o & 0xffu), k6 = static_cast<float>((o >> 8) & 0xffu);
    const float k3 = static_cast<float>((o >> 16) & 0xffu), k7 = static_cast<float>(o >> 24);
    u32x4 v;
    v.x = pk(__builtin_fmaf(k0, s, b), __builtin_fmaf(k1, s, b));
    v.y = pk(__builtin_fmaf(k2, s, b), __builtin_fmaf(k3, s, b));
    v.z = pk(__builtin_fmaf(k4, s, b), __builtin_fmaf(k5, s, b));
    v.w = pk(__builtin_fmaf(k6, s, b), __builtin_fmaf(k7, s, b));
    return as_frag<BF16>(v);
  }
};

// WAVES_M x WAVES_N wavefronts, each WM x WN tiles of 16x16.  BM = WAVES_M*WM*16, BN = WAVES_N*WN*16.
template <typename T, int WAVES_M, int WAVES_N, int WM, int WN, bool HAS_ZP>
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64, 1) w4a16_tile_kernel(TileParams p) {
  constexpr int THREADS = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * WM * 16;
  constexpr int BN = WAVES_N * WN * 16;
  constexpr int BK = 64;                       // k per LDS stage
  constexpr int FRAGS = (BM / 16) * (BK / 32);  // 1 KiB fragments per stage
  constexpr int STAGE_BYTES = FRAGS * 1024;
  constexpr int A_LOADS = BM * BK * 2 / 16 / THREADS;  // 16-byte chunks per thread per stage
  static_assert(BM * BK * 2 / 16 % THREADS == 0, "A tile must split evenly over the threads");

  extern __shared__ __attribute__((aligned(16))) char lds[];  // 2 * STAGE_BYTES

  const int lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15, lq = lane >> 4;
  const uint32_t KT = p.K / 128;

  // ---- XCD-aware tile id: workgroup b runs on XCD b%8; give every XCD a contiguous range of tiles, row tile fastest
  const uint32_t total = p.tiles_m * p.tiles_n;
  uint32_t bid = blockIdx.x;
  {
    const uint32_t per = total / 8, rem = total % 8;
    const uint32_t xcd = bid % 8, local = bid / 8;
    // XCDs 0..rem-1 own per+1 tiles, the rest own per
    bid = xcd * per + (xcd < rem ? xcd : rem) + local;
  }
  const uint32_t tile_n = bid / p.tiles_m, tile_m = bid % p.tiles_m;
  const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

  // ---- A (x) staging: thread t copies chunks q = j*THREADS + t ; row = q / 8, 16-byte chunk c = q % 8 of the row
  const char* a_src[A_LOADS];
  uint32_t a_dst[A_LOADS];
#pragma unroll
  for (int j = 0; j < A_LOADS; ++j) {
    const uint32_t q = j * THREADS + threadIdx.x;
    uint32_t row = q / 8;
    const uint32_t c = q % 8;
    uint32_t grow = m0 + row;
    grow = grow < p.M ? grow : p.M - 1;
    a_src[j] = static_cast<const char*>(p.x) + (static_cast<size_t>(grow) * p.K) * 2 + c * 16;
    a_dst[j] = (((row / 16) * (BK / 32) + c / 4) * 64 + (c % 4) * 16 + row % 16) * 16;
  }

  // ---- weights: this wavefront's WN column tiles
  const uint32_t nt0 = n0 / 16 + wn * WN;
  const u32x4* wsrc = static_cast<const u32x4*>(p.w) + static_cast<size_t>(nt0) * KT * 64 + lane;
  const uint16_t* ssrc = static_cast<const uint16_t*>(p.scales) + static_cast<size_t>(nt0) * KT * 16 + lrow;
  const uint8_t* zsrc = HAS_ZP ? static_cast<const uint8_t*>(p.zeros) + static_cast<size_t>(nt0) * KT * 16 + lrow : nullptr;

  f32x4 acc[WN][WM];
#pragma unroll
  for (int t = 0; t < WN; ++t)
#pragma unroll
    for (int i = 0; i < WM; ++i) acc[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 areg[A_LOADS];
  u32x4 wq[WN];       // current k-tile's packed weights
  u32x4 wq_next[WN];
  uint32_t sc[WN], sc_next[WN], zp[WN], zp_next[WN];

  auto load_a = [&](uint32_t k0) {
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) areg[j] = *reinterpret_cast<const u32x4*>(a_src[j] + static_cast<size_t>(k0) * 2);
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) *reinterpret_cast<u32x4*>(lds + buf * STAGE_BYTES + a_dst[j]) = areg[j];
  };
  auto load_w = [&](u32x4 (&dst)[WN], uint32_t (&s)[WN], uint32_t (&z)[WN], uint32_t kt) {
#pragma unroll
    for (int t = 0; t < WN; ++t) {
      dst[t] = wsrc[(static_cast<size_t>(t) * KT + kt) * 64];
      s[t] = ssrc[(static_cast<size_t>(t) * KT + kt) * 16];
      z[t] = HAS_ZP ? zsrc[(static_cast<size_t>(t) * KT + kt) * 16] : 8u;
    }
  };

  // half = 0/1: which 64-wide half of the current k-tile this stage covers
  auto compute = [&](int buf, int half) {
    const char* abase = lds + buf * STAGE_BYTES + (wm * WM * (BK / 32)) * 1024 + lane * 16;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      typename T::frag bfrag[WN];
#pragma unroll
      for (int t = 0; t < WN; ++t) {
        Dequant<T, HAS_ZP> dq;
        dq.set(sc[t], zp[t]);
        bfrag[t] = dq(wq[t][half * 2 + ks]);
      }
#pragma unroll
      for (int i = 0; i < WM; ++i) {
        const u32x4 a = *reinterpret_cast<const u32x4*>(abase + (i * (BK / 32) + ks) * 1024);
#pragma unroll
        for (int t = 0; t < WN; ++t) acc[t][i] = T::mfma(bfrag[t], as_frag<T>(a), acc[t][i]);
      }
    }
  };

  // ---- pipeline: stage s covers k in [64 s, 64 s + 64); k-tile = s / 2
  const uint32_t stages = p.K / BK;
  load_a(0);
  load_w(wq, sc, zp, 0);
  store_a(0);
  __syncthreads();
  for (uint32_t s = 0; s < stages; ++s) {
    const int buf = s & 1;
    const int half = s & 1;
    if (s + 1 < stages) load_a((s + 1) * BK);
    if (half == 0 && (s >> 1) + 1 < KT) load_w(wq_next, sc_next, zp_next, (s >> 1) + 1);
    compute(buf, half);
    if (s + 1 < stages) store_a(buf ^ 1);
    if (half == 1) {
#pragma unroll
      for (int t = 0; t < WN; ++t) {
        wq[t] = wq_next[t];
        sc[t] = sc_next[t];
        zp[t] = zp_next[t];
      }
    }
    __syncthreads();
  }

  // ---- store: lane holds row m = l%16 of the 16x16 tile and columns 4*(l/16) .. +3
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const uint32_t row = m0 + (wm * WM + i) * 16 + lrow;
    if (row < p.M) {
#pragma unroll
      for (int t = 0; t < WN; ++t) {
        u32x2 o;
        o.x = pack2(T::from_float(acc[t][i][0]), T::from_float(acc[t][i][1]));
        o.y = pack2(T::from_float(acc[t][i][2]), T::from_float(acc[t][i][3]));
        uint16_t* yp = static_cast<uint16_t*>(p.y) + static_cast<size_t>(row) * p.N + (nt0 + t) * 16 + 4 * lq;
        *reinterpret_cast<u32x2*>(yp) = o;
      }
    }
  }
}

}  // namespace ksq
