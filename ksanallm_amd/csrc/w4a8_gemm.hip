// W4A8 (int4 weights, fp16 scales per group of 128 or 64, statically quantized e4m3 activations) GEMM:
//   out[m,n] = alpha * sum_g scale[g,n] * sum_{k in g} a_q[m,k] * w[k,n],      w in -8..7
//
// The fp8 matrix instruction does the products.  An int4 code needs no table to become an e4m3 byte: the byte 0x0u
// (u = w + 8 = 0..15) read as e4m3 is exactly u * 2^-9 (exponent field 0 is the subnormal range m * 2^-9, exponent
// field 1 continues it with (8 + m) * 2^-9), so a packed dword expands into two operand dwords with one shift and two
// ANDs.  The offset goes into the instruction's addend: with xsum[m,g] = sum_{k in g} a_q[m,k],
//   sum_k a_q * (u - 8) * 2^-9 = mfma(u_bytes, a_q, C = -xsum / 64).
// One v_mfma_f32_16x16x128_f8f6f4 spans exactly one scale group of 128 (two of 64: then it is issued once per half,
// the other half's operand bytes cleared); its four results per lane are four consecutive output columns of one token
// and take their four scales in fp32.  The factor 2^9 is folded into alpha.
//
// Packed weight layout: a fragment of 16 weight columns x 128 k is 1 KiB, 16 bytes per lane in lane order; lane l
// (column l % 16, quarter q = l / 16) holds dwords P0..P3, nibble 2j of Pi = u(k = 32q + 8i + j), nibble 2j+1 of
// Pi = u(k = 32q + 8i + 4 + j), j = 0..3.  Fragment (strip, kb) lies at (strip * K/128 + kb) * 1024 bytes.
#include <atomic>

#include "exact_div.h"
#include "ksq_common.h"
#include "splitk_reduce.h"
#include "tile_select.h"
#include "w4a8_tile.h"

namespace ksq {
namespace {

// ------------------------------------------------------------------------------------------------ repack
// src: [K, N/2] bytes, two's-complement nibbles, low nibble = even column (the layout the reference hands to its
// weight preprocessor).  One thread per packed dword.
__global__ void __launch_bounds__(256) w4a8_repack_kernel(const uint8_t* __restrict__ src, uint32_t* __restrict__ dst,
                                                          uint32_t N, uint32_t K) {
  const uint32_t KB = K / 128;
  const size_t t = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;  // one workgroup = one fragment
  const uint32_t frag = blockIdx.x;
  const uint32_t strip = frag / KB, kb = frag % KB;
  const uint32_t l = threadIdx.x >> 2, i = threadIdx.x & 3;
  const uint32_t n = strip * 16 + (l & 15);
  const uint32_t k0 = kb * 128 + (l >> 4) * 32 + i * 8;
  uint32_t w = 0;
#pragma unroll
  for (uint32_t e = 0; e < 8; ++e) {
    const uint32_t k = k0 + e;
    const uint32_t byte = src[static_cast<size_t>(k) * (N / 2) + n / 2];
    const uint32_t u = ((byte >> (4 * (n & 1))) & 15u) ^ 8u;
    const uint32_t pos = e < 4 ? 2 * e : 2 * (e - 4) + 1;
    w |= u << (4 * pos);
  }
  dst[t] = w;
}

// One thread per byte of the [K, N/2] layout.
__global__ void __launch_bounds__(256) w4a8_unpack_kernel(const uint32_t* __restrict__ packed, uint8_t* __restrict__ dst,
                                                          uint32_t N, uint32_t K) {
  const size_t t = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t total = static_cast<size_t>(K) * (N / 2);
  if (t >= total) return;
  const uint32_t k = static_cast<uint32_t>(t / (N / 2));
  const uint32_t nb = static_cast<uint32_t>(t % (N / 2));
  const uint32_t KB = K / 128;
  const uint32_t kb = k / 128, r = k % 128, q = r / 32, i = (r % 32) / 8, e = r % 8;
  const uint32_t pos = e < 4 ? 2 * e : 2 * (e - 4) + 1;
  uint32_t byte = 0;
#pragma unroll
  for (uint32_t h = 0; h < 2; ++h) {
    const uint32_t n = nb * 2 + h;
    const uint32_t l = q * 16 + (n & 15);
    const uint32_t w = packed[(static_cast<size_t>(n / 16) * KB + kb) * 256 + l * 4 + i];
    byte |= ((((w >> (4 * pos)) & 15u) ^ 8u)) << (4 * h);
  }
  dst[t] = static_cast<uint8_t>(byte);
}

// ------------------------------------------------------------------------------------------------ quantizer
__device__ __forceinline__ uint32_t cvt2_sat(float a, float b, uint32_t old, bool hi) {
  float ca = fminf(fmaxf(a, -448.0f), 448.0f);
  float cb = fminf(fmaxf(b, -448.0f), 448.0f);
  ca = (a != a) ? a : ca;
  cb = (b != b) ? b : cb;
  return hi ? static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, static_cast<int>(old), true))
            : static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, static_cast<int>(old), false));
}

// sum of the eight e4m3 values of two dwords, in ascending order
__device__ __forceinline__ float sum8_e4m3(u32x2 q) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q.x), false);
  const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q.x), true);
  const f32x2 c = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q.y), false);
  const f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(q.y), true);
  return ((((((a.x + a.y) + b.x) + b.y) + c.x) + c.y) + d.x) + d.y;
}

// MODE 0: q = e4m3(x / scale[0]); MODE 1: q = e4m3(x / scale[channel]); MODE 2: x is e4m3 already (sums only);
// MODE 3: q = e4m3(x / scale[row]).
// IEEE fp32 division, round to nearest even, saturating.  xsum[g, row] = sum of the 128 quantized values of group g
// (every e4m3 value is a multiple of 2^-9, so the fp32 sum is exact, in any order, while it stays below 2^15).
// Grid: x = chunks of BLOCK * 8 channels, y/z = row; a group of 128 channels is 16 adjacent lanes.
// SG: channels per sum, 128 or 64 (16 or 8 adjacent lanes).
template <typename T, int MODE, int BLOCK, int SG = 128>
__global__ void __launch_bounds__(BLOCK) w4a8_quant_kernel(const void* __restrict__ xin, const float* __restrict__ scale,
                                                         uint8_t* __restrict__ q, float* __restrict__ xsum, uint32_t m,
                                                         uint32_t k) {
  const uint32_t row = blockIdx.z * gridDim.y + blockIdx.y;
  const uint32_t col0 = (blockIdx.x * BLOCK + threadIdx.x) * 8;
  const bool live = row < m && col0 < k;
  const uint32_t t = live ? row : 0;
  const uint32_t col = live ? col0 : 0;
  const size_t e0 = static_cast<size_t>(t) * k + col;
  u32x2 out{0u, 0u};
  if (MODE == 2) {
    out = *reinterpret_cast<const u32x2*>(static_cast<const uint8_t*>(xin) + e0);
  } else {
    const u32x4 raw = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(xin) + e0);
    float v[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[2 * j] = T::lo_to_float(raw[j]);
      v[2 * j + 1] = T::hi_to_float(raw[j]);
    }
    if (MODE == 0 || MODE == 3) {
      // one scale per lane: the quotient from one reciprocal (exact_div.h); an infinite input keeps the division
      const float s = scale[MODE == 3 ? t : 0];
      const ExactDiv div(s);
      // a branch, not a select per element: a select would evaluate the division for every element
      float mx = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) mx = fmaxf(mx, __builtin_fabsf(v[j]));
      if (mx == __builtin_inff()) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = v[j] / s;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = div(v[j]);
      }
    } else {
      const f32x4 s0 = *reinterpret_cast<const f32x4*>(scale + col);
      const f32x4 s1 = *reinterpret_cast<const f32x4*>(scale + col + 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] = v[j] / s0[j];
        v[4 + j] = v[4 + j] / s1[j];
      }
    }
    out.x = cvt2_sat(v[0], v[1], out.x, false);
    out.x = cvt2_sat(v[2], v[3], out.x, true);
    out.y = cvt2_sat(v[4], v[5], out.y, false);
    out.y = cvt2_sat(v[6], v[7], out.y, true);
  }
  float sum = sum8_e4m3(out);
#pragma unroll
  for (int off = 1; off < SG / 8; off <<= 1) sum += __shfl_xor(sum, off, 16);
  if (!live) return;
  if (MODE != 2) *reinterpret_cast<u32x2*>(q + e0) = out;
  if ((threadIdx.x & (SG / 8 - 1)) == 0) xsum[static_cast<size_t>(col / SG) * m + t] = sum;
}

// ------------------------------------------------------------------------------------------------ GEMM
struct W4A8Params {
  const uint8_t* a;      // [M, K] e4m3
  const float* xsum;     // [K/group, M]
  const uint8_t* w;      // packed fragments
  const uint16_t* sc;    // fp16 [K/group, N]
  void* out;             // [M, N]
  uint32_t M, N, K;
  float alpha512;        // alpha * 2^9
};

__device__ __forceinline__ f32x4 mfma_fp8_128(i32x8 a, i32x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

__device__ __forceinline__ i32x8 expand_u4(i32x4 p) {
  i32x8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t w = static_cast<uint32_t>(p[i]);
    r[2 * i] = static_cast<int>(w & 0x0f0f0f0fu);
    r[2 * i + 1] = static_cast<int>((w >> 4) & 0x0f0f0f0fu);
  }
  return r;
}

// Streaming form (HBM-bound at few tokens): a workgroup owns NT strips of 16 weight columns and MT*16 tokens;
// wavefront w takes the k-blocks w, w+WAVES, ... with LOOK of them loaded ahead into registers.  Blocks past the end
// are clamped to the last one and given zero scales, so that control flow stays uniform.  Partials are summed through
// LDS in wavefront order.
// GROUP = 64: the instruction still spans 128 k; it is issued twice per k-block, once with the activation bytes of the
// upper 64 k (lanes 32..63 of the operand) cleared and once with those of the lower 64 k cleared, each with its own
// addend and its own scales - exact, at twice the MFMAs, which a kernel that waits for HBM does not notice.
template <typename TO, int MT, int NT, int WAVES, int LOOK, int GROUP = 128>
__global__ void __launch_bounds__(WAVES * 64) w4a8_splitk_kernel(W4A8Params p) {
  constexpr int GH = 128 / GROUP;  // scale groups per k-block
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lrow = lane & 15;
  const int lq = lane >> 4;
  const uint32_t KB = p.K / 128;
  const uint32_t n0 = blockIdx.x * (16 * NT);
  const uint32_t m0 = blockIdx.y * (16 * MT);

  __shared__ f32x4 red[WAVES][NT][MT][64];

  const uint8_t* wptr = p.w + (static_cast<size_t>(n0 / 16) * KB) * 1024 + lane * 16;
  const uint16_t* scptr = p.sc + n0 + 4 * lq;
  const uint8_t* aptr[MT];
  const float* xsptr[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    uint32_t row = m0 + mt * 16 + lrow;
    row = row < p.M ? row : p.M - 1;  // rows past M repeat the last token; their results are not stored
    aptr[mt] = p.a + static_cast<size_t>(row) * p.K + lq * 32;
    xsptr[mt] = p.xsum + row;
  }

  f32x4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct Stage {
    i32x4 w[NT];
    u32x2 sc[NT][GH];
    i32x4 a0[MT], a1[MT];
    float xs[MT][GH];
  };
  Stage ring[LOOK];
  auto load_stage = [&](Stage& s, uint32_t kb) {
    const bool live = kb < KB;
    kb = live ? kb : KB - 1;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint8_t* wp = wptr + (static_cast<size_t>(nt) * KB + kb) * 1024;
      s.w[nt] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(wp));
#pragma unroll
      for (int h = 0; h < GH; ++h) {
        const u32x2 sc = *reinterpret_cast<const u32x2*>(scptr + (static_cast<size_t>(kb) * GH + h) * p.N + nt * 16);
        s.sc[nt][h] = live ? sc : u32x2{0u, 0u};
      }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const i32x4* ap = reinterpret_cast<const i32x4*>(aptr[mt] + static_cast<size_t>(kb) * 128);
      s.a0[mt] = ap[0];
      s.a1[mt] = ap[1];
#pragma unroll
      for (int h = 0; h < GH; ++h) s.xs[mt][h] = xsptr[mt][(static_cast<size_t>(kb) * GH + h) * p.M];
    }
  };
  auto compute_stage = [&](const Stage& s) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const i32x8 a{s.a0[mt].x, s.a0[mt].y, s.a0[mt].z, s.a0[mt].w, s.a1[mt].x, s.a1[mt].y, s.a1[mt].z, s.a1[mt].w};
#pragma unroll
      for (int h = 0; h < GH; ++h) {
        i32x8 ah = a;
        if (GH == 2) {  // this lane's 32 k lie in half lq / 2 of the k-block
          const int keep = (lq >> 1) == h ? -1 : 0;
#pragma unroll
          for (int e = 0; e < 8; ++e) ah[e] = a[e] & keep;
        }
        const float c = s.xs[mt][h] * -0.015625f;  // -8 * 2^-9 * xsum
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const f32x4 r = mfma_fp8_128(expand_u4(s.w[nt]), ah, f32x4{c, c, c, c});
          acc[nt][mt][0] = __builtin_fmaf(r[0], F16::lo_to_float(s.sc[nt][h].x), acc[nt][mt][0]);
          acc[nt][mt][1] = __builtin_fmaf(r[1], F16::hi_to_float(s.sc[nt][h].x), acc[nt][mt][1]);
          acc[nt][mt][2] = __builtin_fmaf(r[2], F16::lo_to_float(s.sc[nt][h].y), acc[nt][mt][2]);
          acc[nt][mt][3] = __builtin_fmaf(r[3], F16::hi_to_float(s.sc[nt][h].y), acc[nt][mt][3]);
        }
      }
    }
  };

  const uint32_t rounds = (KB + WAVES - 1) / WAVES;
#pragma unroll
  for (int h = 0; h < LOOK; ++h) {
    load_stage(ring[h], wave + h * WAVES);
    __builtin_amdgcn_sched_barrier(0);
  }
  for (uint32_t it = 0; it < rounds; it += LOOK) {
#pragma unroll
    for (int h = 0; h < LOOK; ++h) {
      compute_stage(ring[h]);
      __builtin_amdgcn_sched_barrier(0);
      load_stage(ring[h], wave + (it + h + LOOK) * WAVES);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[wave][nt][mt][lane] = acc[nt][mt];
  __syncthreads();
  for (int idx = threadIdx.x; idx < NT * MT * 64; idx += WAVES * 64) {
    const int l = idx & 63, mt = (idx >> 6) % MT, nt = (idx >> 6) / MT;
    f32x4 v = red[0][nt][mt][l];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) v += red[w][nt][mt][l];
    v *= p.alpha512;
    const uint32_t row = m0 + mt * 16 + (l & 15);
    if (row < p.M) {
      u32x2 o;
      o.x = pack2(TO::from_float(v[0]), TO::from_float(v[1]));
      o.y = pack2(TO::from_float(v[2]), TO::from_float(v[3]));
      uint16_t* yp = static_cast<uint16_t*>(p.out) + static_cast<size_t>(row) * p.N + n0 + nt * 16 + 4 * (l >> 4);
      *reinterpret_cast<u32x2*>(yp) = o;
    }
  }
}

// Measured on MI355X (n = 25600 and n = 5120 at k = 5120, 1 and 16 tokens): the loads of activations, scales and group
// sums are as many as the weight loads of one strip, so a workgroup takes as many strips as still leave the chip half
// covered with workgroups (four strips: 19.2 -> 14.1 us at n = 25600), with no register ring at all - fewer registers,
// more resident wavefronts, and those hide the latency better than a ring does (a ring 2, 3 or 4 deep measured 6-15 %
// slower each step).  Grids below one workgroup per CU split K over eight wavefronts instead of four (n = 5120:
// 8.1 -> 6.1 us).
template <typename TO, int GROUP = 128>
int dispatch_splitk(const W4A8Params& p, hipStream_t s) {
  const SplitKChoice c = select_w4a8_splitk(p.M, p.N);
  const int mt = c.mt, nt = c.nt, waves = c.waves;
  const unsigned groups = p.N / (16 * nt);
  const dim3 grid(groups, static_cast<unsigned>(div_up(p.M, 16 * mt)), 1);
#define KSQ_CASE(MT_, NT_, W_)                                                   \
  if (mt == MT_ && nt == NT_ && waves == W_) {                                   \
    w4a8_splitk_kernel<TO, MT_, NT_, W_, 1, GROUP><<<grid, W_ * 64, 0, s>>>(p);  \
    return KSQ_OK;                                                               \
  }
  KSQ_CASE(1, 1, 4) KSQ_CASE(1, 2, 4) KSQ_CASE(1, 4, 4) KSQ_CASE(2, 1, 4) KSQ_CASE(2, 2, 4) KSQ_CASE(2, 4, 4)
  KSQ_CASE(1, 1, 8) KSQ_CASE(1, 2, 8) KSQ_CASE(1, 4, 8) KSQ_CASE(2, 1, 8) KSQ_CASE(2, 2, 8) KSQ_CASE(2, 4, 8)
#undef KSQ_CASE
  return fail(KSQ_ERR_UNSUPPORTED, "no w4a8 kernel for mt=%d nt=%d waves=%d", mt, nt, waves);
}

// Prefill regime: the MFMA tile kernel of w4a8_tile.h on the grid plan_w4a8_tile lays out (the blockwise-FP8 tile
// shapes; a k-step is one 128-deep group).
template <typename TO, int WM, int GROUP = 128>
int launch_tile(const W4A8Params& q, const TilePlan& plan, float* partial, hipStream_t s) {
  constexpr int kLds = static_cast<int>(w4a8_tile_lds_bytes(WM));
  static std::atomic<uint64_t> configured{0};
  if (int rc = allow_dynamic_lds(configured, reinterpret_cast<const void*>(&w4a8_tile_kernel<TO, WM, GROUP>), kLds)) return rc;
  W4A8TileParams p{};
  p.a = q.a;
  p.xsum = q.xsum;
  p.w = q.w;
  p.sc = q.sc;
  p.out = q.out;
  p.partial = partial;
  p.M = q.M;
  p.N = q.N;
  p.K = q.K;
  p.tiles_m = plan.tiles_m;
  p.tiles_n = plan.tiles_n;
  p.main_items = plan.main_items;
  p.splits = plan.splits;
  p.kb_per_split = plan.kt_per_split;
  p.alpha512 = q.alpha512;
  w4a8_tile_kernel<TO, WM, GROUP><<<plan.grid, 512, kLds, s>>>(p);
  if (plan.splits > 1) {
    const unsigned cut = plan.tiles_m * plan.tiles_n - plan.main_items;
    splitk_reduce_kernel<TO, 32 * WM><<<cut * (4 * WM), 256, 0, s>>>(partial, static_cast<uint16_t*>(p.out), p.M, p.N,
                                                                    p.tiles_m, p.tiles_n, p.main_items, p.splits);
  }
  return KSQ_OK;
}

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT size_t ksq_w4a8_packed_weight_bytes(size_t n, size_t k) { return n * k / 2; }

KSQ_EXPORT int ksq_w4a8_repack_weight(const void* src, void* dst_packed, size_t n, size_t k, void* stream) {
  const char* fn = "ksq_w4a8_repack_weight";
  if (!src || !dst_packed) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (n == 0 || k == 0 || n % 16 != 0 || k % 128 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: n must be a positive multiple of 16 and k of 128 (n=%zu k=%zu)", fn, n, k);
  if (reinterpret_cast<uintptr_t>(dst_packed) & 15u) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: dst must be 16-byte aligned", fn);
  const size_t frags = (n / 16) * (k / 128);
  if (frags > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  w4a8_repack_kernel<<<static_cast<unsigned>(frags), 256, 0, as_stream(stream)>>>(
      static_cast<const uint8_t*>(src), static_cast<uint32_t*>(dst_packed), static_cast<uint32_t>(n), static_cast<uint32_t>(k));
  return check_launch(fn);
}

KSQ_EXPORT int ksq_w4a8_unpack_weight(const void* packed, void* dst, size_t n, size_t k, void* stream) {
  const char* fn = "ksq_w4a8_unpack_weight";
  if (!packed || !dst) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (n == 0 || k == 0 || n % 16 != 0 || k % 128 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: n must be a positive multiple of 16 and k of 128 (n=%zu k=%zu)", fn, n, k);
  const size_t blocks = div_up(k * (n / 2), 256);
  if (blocks > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  w4a8_unpack_kernel<<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(
      static_cast<const uint32_t*>(packed), static_cast<uint8_t*>(dst), static_cast<uint32_t>(n), static_cast<uint32_t>(k));
  return check_launch(fn);
}

KSQ_EXPORT int ksq_w4a8_static_quant(const void* x, const void* scale, void* q, void* xsum, size_t m, size_t k,
                                     int mode, int dtype, void* stream) {
  const char* fn = "ksq_w4a8_static_quant";
  const bool per64 = (mode & KSQ_W4A8_SUMS_PER_64) != 0;  // group sums per 64 channels: what the GEMM with group 64 reads
  mode &= ~KSQ_W4A8_SUMS_PER_64;
  if (!x || !xsum || (mode != KSQ_W4A8_SUMS_ONLY && (!q || !scale))) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (mode != KSQ_W4A8_PER_TENSOR && mode != KSQ_W4A8_PER_CHANNEL && mode != KSQ_W4A8_SUMS_ONLY && mode != KSQ_W4A8_PER_TOKEN)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: unknown mode %d", fn, mode);
  if (k == 0 || k % 128 != 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k must be a positive multiple of 128", fn);
  if (mode != KSQ_W4A8_SUMS_ONLY && dtype != KSQ_F16 && dtype != KSQ_BF16)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  const bool sums = mode == KSQ_W4A8_SUMS_ONLY;
  if ((reinterpret_cast<uintptr_t>(x) & (sums ? 7u : 15u)) || (!sums && (reinterpret_cast<uintptr_t>(q) & 7u)) ||
      (reinterpret_cast<uintptr_t>(xsum) & 3u) || (mode == KSQ_W4A8_PER_CHANNEL && !aligned16(scale)) ||
      ((mode == KSQ_W4A8_PER_TENSOR || mode == KSQ_W4A8_PER_TOKEN) && (reinterpret_cast<uintptr_t>(scale) & 3u)))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: misaligned pointer", fn);
  if (m == 0) return KSQ_OK;
  if (m > 0x7fffffffull || k > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  const unsigned gy = static_cast<unsigned>(m < 32768 ? m : 32768);
  const unsigned gz = static_cast<unsigned>(div_up(m, gy));
  hipStream_t st = as_stream(stream);
  const float* sp = static_cast<const float*>(scale);
  uint8_t* qp = static_cast<uint8_t*>(q);
  float* xs = static_cast<float*>(xsum);
  const uint32_t mm = static_cast<uint32_t>(m), kk = static_cast<uint32_t>(k);
  // the largest block whose chunks tile a row without idle lanes (k is a multiple of 128 = 16 lanes)
  const int block = k % 2048 == 0 ? 256 : (k % 1024 == 0 ? 128 : (k % 512 == 0 || k < 2048 ? 64 : 256));
#define KSQ_Q(TT, MODE_, B_)                                                                                              \
  do {                                                                                                                    \
    const dim3 qgrid(static_cast<unsigned>(div_up(k, B_ * 8)), gy, gz);                                                   \
    if (per64) w4a8_quant_kernel<TT, MODE_, B_, 64><<<qgrid, B_, 0, st>>>(x, sp, qp, xs, mm, kk);                         \
    else w4a8_quant_kernel<TT, MODE_, B_, 128><<<qgrid, B_, 0, st>>>(x, sp, qp, xs, mm, kk);                              \
  } while (0)
#define KSQ_QB(TT, MODE_)                        \
  do {                                           \
    if (block == 256) KSQ_Q(TT, MODE_, 256);     \
    else if (block == 128) KSQ_Q(TT, MODE_, 128);\
    else KSQ_Q(TT, MODE_, 64);                   \
  } while (0)
  if (mode == KSQ_W4A8_SUMS_ONLY) KSQ_QB(F16, 2);
  else if (dtype == KSQ_F16 && mode == KSQ_W4A8_PER_TENSOR) KSQ_QB(F16, 0);
  else if (dtype == KSQ_F16 && mode == KSQ_W4A8_PER_TOKEN) KSQ_QB(F16, 3);
  else if (dtype == KSQ_F16) KSQ_QB(F16, 1);
  else if (mode == KSQ_W4A8_PER_TENSOR) KSQ_QB(BF16, 0);
  else if (mode == KSQ_W4A8_PER_TOKEN) KSQ_QB(BF16, 3);
  else KSQ_QB(BF16, 1);
#undef KSQ_QB
#undef KSQ_Q
  return check_launch(fn);
}

KSQ_EXPORT size_t ksq_w4a8_workspace_size(size_t max_m, size_t n, size_t k) {
  if (n == 0 || k == 0 || k % 128 != 0) return 0;
  // only the split-K form of the tile kernel needs scratch (fp32 partial tiles); the plan is the same for all m of a
  // band of 128 rows
  size_t need = 0;
  for (size_t band_end = 128; max_m > 32; band_end += 128) {
    const size_t m = band_end < max_m ? band_end : max_m;
    const TilePlan t = plan_w4a8_tile(m, n, k);
    need = t.workspace_bytes > need ? t.workspace_bytes : need;
    if (m == max_m) break;
  }
  return need;
}

KSQ_EXPORT int ksq_w4a8_gemm(const void* a_q, const void* xsum, const void* w_packed, const void* scales, float alpha,
                             void* out, size_t m, size_t n, size_t k, size_t group, int out_dtype, void* workspace,
                             size_t workspace_bytes, void* stream) {
  const char* fn = "ksq_w4a8_gemm";
  if (!a_q || !xsum || !w_packed || !scales || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (group != 128 && group != 64) return fail(KSQ_ERR_UNSUPPORTED, "%s: group size %zu (128 or 64)", fn, group);
  if (n == 0 || k == 0 || n % 16 != 0 || k % 128 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: n must be a positive multiple of 16 and k of 128 (n=%zu k=%zu)", fn, n, k);
  if (out_dtype != KSQ_F16 && out_dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: out dtype must be f16 or bf16", fn);
  if (!aligned16(a_q) || !aligned16(w_packed) || !aligned16(scales) || !aligned16(out) || !aligned16(xsum))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: every pointer must be 16-byte aligned", fn);
  if (m == 0) return KSQ_OK;
  if (m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull || div_up(m, 16) > 65535)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  W4A8Params p{};
  p.a = static_cast<const uint8_t*>(a_q);
  p.xsum = static_cast<const float*>(xsum);
  p.w = static_cast<const uint8_t*>(w_packed);
  p.sc = static_cast<const uint16_t*>(scales);
  p.out = out;
  p.M = static_cast<uint32_t>(m);
  p.N = static_cast<uint32_t>(n);
  p.K = static_cast<uint32_t>(k);
  p.alpha512 = alpha * 512.0f;
  hipStream_t st = as_stream(stream);
  int rc;
  if (group == 64) {
    // two scale groups per k-block: the streaming kernel, or 128-token tiles over all of K (no workspace)
    if (use_w4a8_tile(m, n, k)) {
      if (256 * k > 0xffffffffull || 16 * (k / 128) * 1024 > 0xffffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k too large", fn);
      TilePlan plan{};
      plan.block_m = 128;
      plan.tiles_m = static_cast<unsigned>(div_up(m, 128));
      plan.tiles_n = static_cast<unsigned>(div_up(n, 256));
      plan.main_items = 0;
      plan.splits = 1;
      plan.kt_per_split = static_cast<unsigned>(k / 128);
      plan.grid = plan.tiles_m * plan.tiles_n;
      rc = out_dtype == KSQ_F16 ? launch_tile<F16, 4, 64>(p, plan, nullptr, st) : launch_tile<BF16, 4, 64>(p, plan, nullptr, st);
    } else {
      rc = out_dtype == KSQ_F16 ? dispatch_splitk<F16, 64>(p, st) : dispatch_splitk<BF16, 64>(p, st);
    }
  } else if (use_w4a8_tile(m, n, k)) {
    const TilePlan plan = plan_w4a8_tile(m, n, k);
    if (plan.splits > 1 && (!workspace || workspace_bytes < plan.workspace_bytes || !aligned16(workspace)))
      return fail(KSQ_ERR_WORKSPACE, "%s: m=%zu n=%zu k=%zu needs %zu bytes of 16-byte aligned workspace, got %zu", fn, m,
                  n, k, plan.workspace_bytes, workspace ? workspace_bytes : size_t(0));
    if (256 * k > 0xffffffffull || 16 * (k / 128) * 1024 > 0xffffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k too large", fn);
    float* partial = plan.splits > 1 ? static_cast<float*>(workspace) : nullptr;
    if (plan.block_m == 128)
      rc = out_dtype == KSQ_F16 ? launch_tile<F16, 4>(p, plan, partial, st) : launch_tile<BF16, 4>(p, plan, partial, st);
    else
      rc = out_dtype == KSQ_F16 ? launch_tile<F16, 8>(p, plan, partial, st) : launch_tile<BF16, 8>(p, plan, partial, st);
  } else {
    rc = out_dtype == KSQ_F16 ? dispatch_splitk<F16>(p, st) : dispatch_splitk<BF16>(p, st);
  }
  if (rc != KSQ_OK) return rc;
  return check_launch(fn);
}
