// Blockwise-scaled FP8 (OCP e4m3) GEMM:  out[m,n] = sum_kb (a_q[m,kb] . b[n,kb]) * a_s[kb,m] * b_s[n/128,kb]
//
// Both operands are K-contiguous bytes, which is what v_mfma_f32_16x16x128_f8f6f4 wants: lane l supplies the 32
// bytes k = 32*(l/16) .. +31 of row l%16.  Weights are the row operand, activations the column operand, so a lane's
// four results are four consecutive output columns of one token.
#include <atomic>
#include <cstdio>
#include <cstdlib>

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

// Decode regime (HBM-bound): a workgroup owns 16 weight rows and MT*16 tokens; wavefront w takes the 128-wide
// k-blocks w, w+WAVES, ... and keeps LOOK of them in flight (a ring of register stages, refilled in place right after
// use; blocks past the end are clamped to the last one and given a zero scale, so that control flow stays uniform and
// the compiler's wait counts stay exact).  Partials are summed through LDS in wavefront order.
template <typename TO, int MT, int NT, int WAVES, int LOOK>
__global__ void __launch_bounds__(WAVES * 64) fp8_splitk_kernel(Fp8Params p) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lrow = lane & 15;
  const int lq = lane >> 4;
  const uint32_t KB = p.K / 128;
  const uint32_t n0 = blockIdx.x * (16 * NT);  // NT strips of 16 weight rows share every activation fragment
  const uint32_t m0 = blockIdx.y * (16 * MT);

  __shared__ f32x4 red[WAVES][NT][MT][64];

  const uint8_t* bptr = p.b + static_cast<size_t>(n0 + lrow) * p.K + lq * 32;
  const float* bs = p.b_s + static_cast<size_t>(n0 / 128) * KB;  // 16*NT <= 128 rows: one scale block
  const uint8_t* aptr[MT];
  const float* asptr[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    uint32_t row = m0 + mt * 16 + lrow;
    row = row < p.M ? row : p.M - 1;  // rows past M repeat the last token; their results are not stored
    aptr[mt] = p.a + static_cast<size_t>(row) * p.K + lq * 32;
    asptr[mt] = p.a_s + row;
  }

  f32x4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct Stage {
    i32x4 w0[NT], w1[NT];
    i32x4 a0[MT], a1[MT];
    float as[MT];
    float ws;
  };
  Stage ring[LOOK];
  auto load_stage = [&](Stage& s, uint32_t kb) {
    const bool live = kb < KB;
    kb = live ? kb : KB - 1;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const i32x4* wp = reinterpret_cast<const i32x4*>(bptr + static_cast<size_t>(nt) * 16 * p.K + static_cast<size_t>(kb) * 128);
      s.w0[nt] = __builtin_nontemporal_load(wp);
      s.w1[nt] = __builtin_nontemporal_load(wp + 1);
    }
    s.ws = live ? bs[kb] : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const i32x4* ap = reinterpret_cast<const i32x4*>(aptr[mt] + static_cast<size_t>(kb) * 128);
      s.a0[mt] = ap[0];
      s.a1[mt] = ap[1];
      s.as[mt] = asptr[mt][static_cast<size_t>(kb) * p.M];
    }
  };
  auto compute_stage = [&](const Stage& s) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const i32x8 a{s.a0[mt].x, s.a0[mt].y, s.a0[mt].z, s.a0[mt].w, s.a1[mt].x, s.a1[mt].y, s.a1[mt].z, s.a1[mt].w};
      const float sc = s.as[mt] * s.ws;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const i32x8 w{s.w0[nt].x, s.w0[nt].y, s.w0[nt].z, s.w0[nt].w, s.w1[nt].x, s.w1[nt].y, s.w1[nt].z, s.w1[nt].w};
        const f32x4 r = mfma_fp8_128(w, a, f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[nt][mt][i] = __builtin_fmaf(r[i], sc, acc[nt][mt][i]);
      }
    }
  };

  const uint32_t rounds = (KB + WAVES - 1) / WAVES;  // k-blocks this wavefront may own
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

template <typename TO, int MT, int NT, int WAVES, int LOOK>
void launch_splitk(const Fp8Params& p, hipStream_t s) {
  dim3 grid(p.N / (16 * NT), static_cast<unsigned>(div_up(p.M, 16 * MT)), 1);
  fp8_splitk_kernel<TO, MT, NT, WAVES, LOOK><<<grid, WAVES * 64, 0, s>>>(p);
}

template <typename TO>
int dispatch(const Fp8Params& p, hipStream_t s) {
  const int mt = p.M <= 16 ? 1 : 2;
  // Measured on MI355X: four wavefronts per workgroup with a shallow ring stream fastest (the grid already holds
  // thousands of wavefronts; deeper rings only cost registers, i.e. resident wavefronts).
  // the activation fragments are as large as the weight fragments: two strips share them once there are several
  // tokens, or when K is the long dimension (few strips, long streams)
  int nt = (p.M > 8 || p.K > p.N) ? 2 : 1;
  if (p.N % (16 * nt) != 0) nt = 1;
#define KSQ_CASE(MT_, NT_) \
  if (mt == MT_ && nt == NT_) { launch_splitk<TO, MT_, NT_, 4, 2>(p, s); return KSQ_OK; }
  KSQ_CASE(1, 1) KSQ_CASE(1, 2) KSQ_CASE(2, 1) KSQ_CASE(2, 2)
#undef KSQ_CASE
  return fail(KSQ_ERR_UNSUPPORTED, "no fp8 decode kernel for mt=%d nt=%d", mt, nt);
}

}  // namespace
}  // namespace ksq

namespace ksq {
namespace {

template <typename TO>
int launch_fp8_tile(const Fp8Params& q, const TilePlan& plan, float* partial, hipStream_t s) {
  // two operand stages, two stages of activation scales, the weight scales of the k range
  constexpr int kLdsMax = 160 * 1024;
  const size_t kb_max = (plan.main_items || plan.splits == 1) ? q.K / 128 : plan.kt_per_split;  // whole tiles span all of K
  const size_t lds = 2 * 32 * 2048 + 2 * 1024 + 2 * kb_max * 4;
  if (lds > kLdsMax) return fail(KSQ_ERR_UNSUPPORTED, "k range of %zu blocks per workgroup does not fit the LDS", kb_max);
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
  p.main_items = plan.main_items;
  p.splits = plan.splits;
  p.kb_per_split = plan.kt_per_split;
  fp8_tile_kernel<TO><<<plan.grid, 512, lds, s>>>(p);
  if (plan.splits > 1) {
    const unsigned cut = plan.tiles_m * plan.tiles_n - plan.main_items;
    splitk_reduce_kernel<TO, 256><<<cut * 32, 256, 0, s>>>(partial, static_cast<uint16_t*>(p.out), p.M, p.N, p.tiles_m, p.tiles_n,
                                                          p.main_items, p.splits);
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
  // the plan is the same for all m of a band of 256 rows
  for (size_t band_end = 256; max_m > 32; band_end += 256) {
    const size_t m = band_end < max_m ? band_end : max_m;
    const TilePlan t = plan_fp8_tile(m, n, k);
    need = t.workspace_bytes > need ? t.workspace_bytes : need;
    if (m == max_m) break;
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
