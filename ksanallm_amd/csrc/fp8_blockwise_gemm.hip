// Blockwise-scaled FP8 (OCP e4m3) GEMM:  out[m,n] = sum_kb (a_q[m,kb] . b[n,kb]) * a_s[kb,m] * b_s[n/128,kb]
//
// Both operands are K-contiguous bytes, which is what v_mfma_f32_16x16x128_f8f6f4 wants: lane l supplies the 32
// bytes k = 32*(l/16) .. +31 of row l%16.  Weights are the row operand, activations the column operand, so a lane's
// four results are four consecutive output columns of one token.
#include <atomic>

#include "fp8_tile.h"
#include "ksq_common.h"
#include "splitk_reduce.h"
#include "tile_select.h"

namespace ksq {
namespace {

struct Fp8Params {
  const uint8_t* a;   // [m, k]
  const float* a_s;   // [k/128, m]
  const uint8_t* b;   // [n, k]
  const float* b_s;   // [ceil(n/128), k/128]
  void* out;          // [m, n]
  uint32_t M, N, K;
};

__device__ __forceinline__ f32x4 mfma_fp8_128(i32x8 a, i32x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

__device__ __forceinline__ i32x8 load32(const uint8_t* p) {
  i32x4 lo = *reinterpret_cast<const i32x4*>(p);
  i32x4 hi = *reinterpret_cast<const i32x4*>(p + 16);
  return i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
}

// Decode regime: a workgroup owns 16 weight rows and MT*16 tokens; wavefront w takes the 128-wide k-blocks
// w, w+WAVES, ...; partials are summed through LDS in wavefront order.
template <typename TO, int MT, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) fp8_splitk_kernel(Fp8Params p) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int lrow = lane & 15;
  const int lq = lane >> 4;
  const uint32_t KB = p.K / 128;
  const uint32_t n0 = blockIdx.x * 16;
  const uint32_t m0 = blockIdx.y * (16 * MT);

  __shared__ f32x4 red[WAVES][MT][64];

  const uint8_t* bptr = p.b + static_cast<size_t>(n0 + lrow) * p.K + lq * 32;
  const float* bs = p.b_s + static_cast<size_t>(n0 / 128) * KB;
  const uint8_t* aptr[MT];
  uint32_t arow[MT];
  bool ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    arow[mt] = m0 + mt * 16 + lrow;
    ok[mt] = arow[mt] < p.M;
    aptr[mt] = p.a + static_cast<size_t>(ok[mt] ? arow[mt] : 0) * p.K + lq * 32;
  }

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct Stage {
    i32x8 w;
    i32x8 a[MT];
    float sc[MT];
  };
  auto load_stage = [&](Stage& s, uint32_t kb) {
    const i32x4* wp = reinterpret_cast<const i32x4*>(bptr + static_cast<size_t>(kb) * 128);
    i32x4 lo = __builtin_nontemporal_load(wp), hi = __builtin_nontemporal_load(wp + 1);
    s.w = i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    const float wsc = bs[kb];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (ok[mt]) {
        s.a[mt] = load32(aptr[mt] + static_cast<size_t>(kb) * 128);
        s.sc[mt] = p.a_s[static_cast<size_t>(kb) * p.M + arow[mt]] * wsc;
      } else {
        s.a[mt] = i32x8{0, 0, 0, 0, 0, 0, 0, 0};
        s.sc[mt] = 0.f;
      }
    }
  };
  auto compute_stage = [&](const Stage& s) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f32x4 r = mfma_fp8_128(s.w, s.a[mt], f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[mt][i] += r[i] * s.sc[mt];
    }
  };

  uint32_t kb = wave;
  if (kb < KB) {
    Stage cur;
    load_stage(cur, kb);
    for (;;) {
      uint32_t nk = kb + WAVES;
      if (nk < KB) {
        Stage nxt;
        load_stage(nxt, nk);
        compute_stage(cur);
        cur = nxt;
        kb = nk;
      } else {
        compute_stage(cur);
        break;
      }
    }
  }

#pragma unroll
  for (int mt = 0; mt < MT; ++mt) red[wave][mt][lane] = acc[mt];
  __syncthreads();
  for (int idx = threadIdx.x; idx < MT * 64; idx += WAVES * 64) {
    const int l = idx & 63, mt = idx >> 6;
    f32x4 v = red[0][mt][l];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) v += red[w][mt][l];
    const uint32_t row = m0 + mt * 16 + (l & 15);
    if (row < p.M) {
      u32x2 o;
      o.x = pack2(TO::from_float(v[0]), TO::from_float(v[1]));
      o.y = pack2(TO::from_float(v[2]), TO::from_float(v[3]));
      uint16_t* yp = static_cast<uint16_t*>(p.out) + static_cast<size_t>(row) * p.N + n0 + 4 * (l >> 4);
      *reinterpret_cast<u32x2*>(yp) = o;
    }
  }
}

template <typename TO>
int dispatch(const Fp8Params& p, hipStream_t s) {
  const uint32_t KB = p.K / 128;
  const int mt = p.M <= 16 ? 1 : (p.M <= 32 ? 2 : 4);
  const bool w16 = KB >= 64 && mt < 4;
  dim3 grid(p.N / 16, static_cast<unsigned>(div_up(p.M, 16 * mt)), 1);
  if (mt == 1) {
    if (w16) fp8_splitk_kernel<TO, 1, 16><<<grid, 1024, 0, s>>>(p);
    else fp8_splitk_kernel<TO, 1, 8><<<grid, 512, 0, s>>>(p);
  } else if (mt == 2) {
    if (w16) fp8_splitk_kernel<TO, 2, 16><<<grid, 1024, 0, s>>>(p);
    else fp8_splitk_kernel<TO, 2, 8><<<grid, 512, 0, s>>>(p);
  } else {
    fp8_splitk_kernel<TO, 4, 8><<<grid, 512, 0, s>>>(p);
  }
  return KSQ_OK;
}

template <typename TO>
int launch_fp8_tile(const Fp8Params& q, const TilePlan& plan, float* partial, hipStream_t s) {
  // two operand stages, two stages of activation scales, the weight scales of the k range
  constexpr int kLdsMax = 160 * 1024;
  const size_t lds = 2 * 32 * 2048 + 2 * 1024 + 2 * static_cast<size_t>(plan.kt_per_split) * 4;
  if (lds > kLdsMax) return fail(KSQ_ERR_UNSUPPORTED, "k range of %u blocks per workgroup does not fit the LDS", plan.kt_per_split);
  static std::atomic<bool> configured{false};
  if (!configured.load(std::memory_order_acquire)) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&fp8_tile_kernel<TO>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax);
    if (e != hipSuccess) return fail(KSQ_ERR_LAUNCH, "hipFuncSetAttribute(LDS %d): %s", kLdsMax, hipGetErrorString(e));
    configured.store(true, std::memory_order_release);
  }
  Fp8TileParams p{};
  p.a = q.a;
  p.a_s = q.a_s;
  p.b = q.b;
  p.b_s = q.b_s;
  p.out = q.out;
  p.partial = partial;
  p.M = q.M;
  p.N = q.N;
  p.K = q.K;
  p.tiles_m = plan.tiles_m;
  p.tiles_n = plan.tiles_n;
  p.splits = plan.splits;
  p.kb_per_split = plan.kt_per_split;
  fp8_tile_kernel<TO><<<plan.tiles_m * plan.tiles_n * plan.splits, 512, lds, s>>>(p);
  if (plan.splits > 1) {
    const size_t mn = static_cast<size_t>(p.M) * p.N;
    splitk_reduce_kernel<TO><<<static_cast<unsigned>(div_up(mn, 256 * 8)), 256, 0, s>>>(partial, static_cast<uint16_t*>(p.out), mn,
                                                                                   plan.splits);
  }
  return KSQ_OK;
}

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT size_t ksq_fp8_blockwise_workspace_size(size_t max_m, size_t n, size_t k) {
  // only the split-K form of the tile kernel needs scratch: fp32 partial tiles
  if (n == 0 || k == 0 || k % 128 != 0) return 0;
  size_t need = 0;
  for (size_t m = 65; m <= max_m; ++m) {
    const TilePlan t = plan_fp8_tile(m, n, k);
    if (t.splits == 1 && m % 256 == 0) break;  // the grid only grows from here on
    need = t.workspace_bytes > need ? t.workspace_bytes : need;
  }
  return need;
}

KSQ_EXPORT int ksq_fp8_blockwise_gemm(const void* a_q, const void* a_s, const void* b, const void* b_s, void* out,
                                      size_t m, size_t n, size_t k, int out_dtype, void* workspace,
                                      size_t workspace_bytes, void* stream) {
  const char* fn = "ksq_fp8_blockwise_gemm";
  if (!a_q || !a_s || !b || !b_s || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (!aligned16(a_q) || !aligned16(b) || !aligned16(out) || (reinterpret_cast<uintptr_t>(a_s) & 3u) ||
      (reinterpret_cast<uintptr_t>(b_s) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: a_q, b, out must be 16-byte aligned, scales 4-byte aligned", fn);
  if (n == 0 || k == 0 || k % 128 != 0 || n % 16 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need k %% 128 == 0 and n %% 16 == 0 (n=%zu k=%zu)", fn, n, k);
  if (out_dtype != KSQ_F16 && out_dtype != KSQ_BF16)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: output dtype must be f16 or bf16", fn);
  if (m == 0) return KSQ_OK;
  if (m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: dimension too large", fn);
  if (div_up(m, 16) > 65535) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: m too large", fn);
  Fp8Params p{static_cast<const uint8_t*>(a_q), static_cast<const float*>(a_s), static_cast<const uint8_t*>(b),
              static_cast<const float*>(b_s), out, static_cast<uint32_t>(m), static_cast<uint32_t>(n),
              static_cast<uint32_t>(k)};
  int rc;
  if (use_fp8_tile(m, n, k)) {
    const TilePlan plan = plan_fp8_tile(m, n, k);
    if (plan.splits > 1 && (!workspace || workspace_bytes < plan.workspace_bytes || !aligned16(workspace)))
      return fail(KSQ_ERR_WORKSPACE, "%s: m=%zu n=%zu k=%zu needs %zu bytes of 16-byte aligned workspace, got %zu", fn, m,
                  n, k, plan.workspace_bytes, workspace ? workspace_bytes : size_t(0));
    if (256 * k > 0xffffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k too large", fn);
    float* partial = plan.splits > 1 ? static_cast<float*>(workspace) : nullptr;
    rc = out_dtype == KSQ_F16 ? launch_fp8_tile<F16>(p, plan, partial, as_stream(stream))
                              : launch_fp8_tile<BF16>(p, plan, partial, as_stream(stream));
  } else {
    rc = out_dtype == KSQ_F16 ? dispatch<F16>(p, as_stream(stream)) : dispatch<BF16>(p, as_stream(stream));
  }
  if (rc) return rc;
  return check_launch(fn);
}
