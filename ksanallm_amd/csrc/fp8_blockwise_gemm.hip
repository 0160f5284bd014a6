// Blockwise-scaled FP8 (OCP e4m3) GEMM:  out[m,n] = sum_kb (a_q[m,kb] . b[n,kb]) * a_s[kb,m] * b_s[n/128,kb]
//
// v_mfma_f32_16x16x128_f8f6f4 wants from lane l the 32 bytes k = 32*(l/16) .. +31 of row l%16.  Activations are read
// from their row-major [m, k] bytes; weights come in the packed fragment layout (ksq_fp8_repack_weight): a fragment of
// 16 weight rows x 128 k is 2 KiB, two 1 KiB halves of 16 bytes per lane in lane order, so that every wavefront load is
// one contiguous KiB (rows of the checkpoint layout lie K bytes apart, and 16-byte pieces of 16 different rows per
// load run the memory pipeline at a quarter of its rate: 52 % of the HBM rate against 75-80 % from fragments).
// Weights are the row operand, activations the column operand, so a lane's four results are four consecutive output
// columns of one token.
#include <atomic>
#include <cstdio>
#include <cstdlib>

#include "fp8_tile.h"
#include <algorithm>

#include "ksq_common.h"
#include "splitk_reduce.h"
#include "tile_select.h"

namespace ksq {
namespace {

struct Fp8Params {
  const uint8_t* a;   // [m, k]
  const float* a_s;   // [k/128, m]
  const uint8_t* b;   // [n, k] in 2 KiB fragments (ksq_fp8_repack_weight)
  const float* b_s;   // [ceil(n/128), k/128]
  void* out;          // [m, n]
  uint32_t M, N, K;
  float* out32;       // dense form, verification only: the fp32 sums go here, [m, n], and nothing is rounded to TO
  uint32_t as_row_stride, as_kb_stride;  // a_s[row * as_row_stride + kb * as_kb_stride]: (1, M) in the dense form
  // grouped (MoE) form: row block b holds the slots sorted_ids[b*16*MT ..] of expert expert_ids[b]
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_w;
  uint32_t numel, top_k, scale_rows;  // scale_rows = ceil(N/128): rows of one expert's b_s
  // Grouped form for a handful of slots (sorted_ids == nullptr): expert_ids holds the router's ids [numel] as they are
  // and block b is slot b alone (row b / top_k of a, expert expert_ids[b], output row b; an id outside
  // [0, num_experts) leaves the row unwritten).  TOKSUM instances: block b is token b, whose top_k rows of a
  // [numel, kb_per_expert * 128] lie one behind the other as one row of K = top_k * kb_per_expert * 128 values; k-block
  // kb of it meets k-block kb % kb_per_expert of expert expert_ids[b * top_k + kb / kb_per_expert], the weight scale
  // times the routing weight topk_w[...]; the fp32 sum over all of K is output row b of [tokens, N].
  uint32_t num_experts, kb_per_expert;
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
// GROUPED: the MoE form.  Row block blockIdx.y is one block of the aligned slot permutation: slot s reads activation
// row s / top_k (pad slots carry s >= numel), the weights and weight scales are those of expert expert_ids[block], the
// result goes to out[s, :] (times topk_w[s] when given).  Blocks past num_post_pad leave at once.
template <typename TO, int MT, int NT, int WAVES, int LOOK, bool GROUPED = false, bool TOKSUM = false>
__global__ void __launch_bounds__(WAVES * 64) fp8_splitk_kernel(Fp8Params p) {
  static_assert(!TOKSUM || (GROUPED && MT == 1), "the token-sum form is a grouped decode form");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lrow = lane & 15;
  const int lq = lane >> 4;
  const uint32_t KB = TOKSUM ? p.kb_per_expert : p.K / 128;  // k-blocks of a weight strip
  const uint32_t KBL = p.K / 128;                            // k-blocks of a row of a
  const uint32_t n0 = blockIdx.x * (16 * NT);  // NT strips of 16 weight rows share every activation fragment
  const uint32_t m0 = blockIdx.y * (16 * MT);

  __shared__ f32x4 red[WAVES][NT][MT][64];
  __shared__ uint32_t tok_ids[TOKSUM ? 32 : 1];
  __shared__ float tok_w[TOKSUM ? 32 : 1];

  const bool few = GROUPED && p.sorted_ids == nullptr;  // a handful of slots: one per block, no aligned permutation
  size_t expert = 0;
  if (GROUPED) {
    if (TOKSUM) {
      if (threadIdx.x < p.top_k) {
        tok_ids[threadIdx.x] = static_cast<uint32_t>(p.expert_ids[blockIdx.y * p.top_k + threadIdx.x]);
        tok_w[threadIdx.x] = p.topk_w ? p.topk_w[blockIdx.y * p.top_k + threadIdx.x] : 1.0f;
      }
      __syncthreads();
    } else {
      if (!few && m0 >= static_cast<uint32_t>(p.num_post_pad[0])) return;  // uniform: the whole workgroup leaves
      const uint32_t e = static_cast<uint32_t>(p.expert_ids[blockIdx.y]);
      if (few && e >= p.num_experts) return;
      expert = e;
    }
  }
  // fragment (strip, k-block) at ((expert*N/16 + strip)*KB + kb) * 2048; this lane's two 16-byte halves at 16*lane, +1024
  const uint8_t* bptr = p.b + ((expert * (p.N / 16) + n0 / 16) * KB) * 2048 + lane * 16;
  const float* bs = p.b_s + (expert * p.scale_rows + n0 / 128) * KB;  // 16*NT <= 128 rows: one scale block
  const uint8_t* aptr[MT];
  const float* asptr[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    uint32_t row = m0 + mt * 16 + lrow;
    if (few || TOKSUM) {
      // every lane reads the block's one row (their results are not stored)
      row = TOKSUM ? blockIdx.y : blockIdx.y / p.top_k;
    } else if (GROUPED) {
      uint32_t sid = static_cast<uint32_t>(p.sorted_ids[row]);
      sid = sid < p.numel ? sid : p.numel - 1;  // pad slots read some valid row; their results are not stored
      row = sid / p.top_k;
    } else {
      row = row < p.M ? row : p.M - 1;  // rows past M repeat the last token; their results are not stored
    }
    aptr[mt] = p.a + static_cast<size_t>(row) * p.K + lq * 32;
    asptr[mt] = p.a_s + static_cast<size_t>(row) * p.as_row_stride;
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
    bool live = kb < KBL;
    kb = live ? kb : KBL - 1;
    uint32_t kbw = kb;           // k-block inside the weight strip
    const uint8_t* wbase = bptr;
    const float* sbase = bs;
    float rw = 1.0f;
    if constexpr (TOKSUM) {
      // the expert whose strip this k-block of the token's row meets (wave-uniform: scalar address arithmetic)
      const uint32_t j = kb / KB;
      kbw = kb - j * KB;
      const uint32_t e = __builtin_amdgcn_readfirstlane(tok_ids[j]);
      rw = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, tok_w[j])));
      live = live && e < p.num_experts;
      const size_t e_ok = e < p.num_experts ? e : 0;
      wbase = bptr + (e_ok * (p.N / 16) * KB) * 2048;
      sbase = bs + e_ok * p.scale_rows * KB;
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint8_t* wp = wbase + (static_cast<size_t>(nt) * KB + kbw) * 2048;
      s.w0[nt] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(wp));
      s.w1[nt] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(wp + 1024));
    }
    s.ws = live ? sbase[kbw] * rw : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const i32x4* ap = reinterpret_cast<const i32x4*>(aptr[mt] + static_cast<size_t>(kb) * 128);
      s.a0[mt] = ap[0];
      s.a1[mt] = ap[1];
      s.as[mt] = asptr[mt][static_cast<size_t>(kb) * p.as_kb_stride];
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

  const uint32_t rounds = (KBL + WAVES - 1) / WAVES;  // k-blocks this wavefront may own
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
  // Grouped form: the slot ids and routing weights of this lane's rows, fetched before the first store.  Read next to
  // each store they would wait for the stores in front of them (the compiler cannot know that the output does not
  // overlap the index arrays), one memory round trip after the other.
  static_assert(MT <= 2, "the epilogue selects between two row tiles");
  uint32_t esid0 = 0, esid1 = 0;
  float erw0 = 1.0f, erw1 = 1.0f;
  if (few || TOKSUM) {
    esid0 = (lane & 15) == 0 ? blockIdx.y : 0xffffffffu;  // the block's one row; the others are not stored
    esid1 = 0xffffffffu;
    if (!TOKSUM && p.topk_w && esid0 < p.numel) erw0 = p.topk_w[esid0];
  } else if (GROUPED) {
    esid0 = static_cast<uint32_t>(p.sorted_ids[m0 + (lane & 15)]);
    if (MT > 1) esid1 = static_cast<uint32_t>(p.sorted_ids[m0 + 16 + (lane & 15)]);
    if (p.topk_w) {
      if (esid0 < p.numel) erw0 = p.topk_w[esid0];
      if (MT > 1 && esid1 < p.numel) erw1 = p.topk_w[esid1];
    }
  }
  for (int idx = threadIdx.x; idx < NT * MT * 64; idx += WAVES * 64) {
    const int l = idx & 63, mt = (idx >> 6) % MT, nt = (idx >> 6) / MT;
    f32x4 v = red[0][nt][mt][l];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) v += red[w][nt][mt][l];
    uint32_t row = m0 + mt * 16 + (l & 15);
    bool live = row < p.M;
    if (GROUPED) {
      const uint32_t sid = mt ? esid1 : esid0;
      live = sid < p.numel;
      row = sid;
      v *= mt ? erw1 : erw0;
    }
    if (live && !GROUPED && p.out32) {
      *reinterpret_cast<f32x4*>(p.out32 + static_cast<size_t>(row) * p.N + n0 + nt * 16 + 4 * (l >> 4)) = v;
    } else if (live) {
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

// grouped (MoE) form: one row block of the aligned permutation per blockIdx.y
template <typename TO>
int dispatch_grouped(const Fp8Params& p, int mt, unsigned blocks, hipStream_t s) {
  // four strips per workgroup share the gathered activation fragments (measured: 5-12 % faster than two)
  const int nt = p.N % 64 == 0 ? 4 : (p.N % 32 == 0 ? 2 : 1);
#define KSQ_CASE(MT_, NT_)                                                             \
  if (mt == MT_ && nt == NT_) {                                                        \
    dim3 grid(p.N / (16 * NT_), blocks, 1);                                            \
    fp8_splitk_kernel<TO, MT_, NT_, 4, 2, true><<<grid, 4 * 64, 0, s>>>(p);            \
    return KSQ_OK;                                                                     \
  }
  KSQ_CASE(1, 1) KSQ_CASE(1, 2) KSQ_CASE(1, 4) KSQ_CASE(2, 1) KSQ_CASE(2, 2) KSQ_CASE(2, 4)
#undef KSQ_CASE
  return fail(KSQ_ERR_UNSUPPORTED, "no grouped fp8 kernel for mt=%d nt=%d", mt, nt);
}

template <typename TO>
int dispatch(const Fp8Params& p, hipStream_t s) {
  const int mt = p.M <= 16 ? 1 : 2;
  // Measured on MI355X: four wavefronts per workgroup with a shallow ring stream fastest (the grid already holds
  // thousands of wavefronts; deeper rings only cost registers, i.e. resident wavefronts).
  // the activation fragments are as large as the weight fragments: two strips share them once there are several
  // tokens, or when K is the long dimension (few strips, long streams)
  int nt = (p.M > 8 || p.K > p.N) ? 2 : 1;
  // several blocks of 32 tokens (small problems above 32 tokens): four strips share a block's activation fragments while
  // the blocks together still give every other CU a workgroup
  if (p.M > 32 && p.N % 64 == 0 && p.N / 64 * div_up(p.M, 32) >= 128) nt = 4;
  if (p.N % (16 * nt) != 0) nt = 1;
#define KSQ_CASE(MT_, NT_) \
  if (mt == MT_ && nt == NT_) { launch_splitk<TO, MT_, NT_, 4, 2>(p, s); return KSQ_OK; }
  KSQ_CASE(1, 1) KSQ_CASE(1, 2) KSQ_CASE(2, 1) KSQ_CASE(2, 2) KSQ_CASE(2, 4)
#undef KSQ_CASE
  return fail(KSQ_ERR_UNSUPPORTED, "no fp8 decode kernel for mt=%d nt=%d", mt, nt);
}

}  // namespace
}  // namespace ksq

namespace ksq {
namespace {

template <typename TO, int WM>
int launch_fp8_tile(const Fp8Params& q, const TilePlan& plan, float* partial, hipStream_t s) {
  // two operand stages, two stages of activation scales, the weight scales of the k range
  constexpr int kLdsMax = 160 * 1024;
  const size_t kb_max = (plan.main_items || plan.splits == 1) ? q.K / 128 : plan.kt_per_split;  // whole tiles span all of K
  const size_t lds = fp8_tile_lds_bytes(WM, kb_max);
  if (lds > kLdsMax) return fail(KSQ_ERR_UNSUPPORTED, "k range of %zu blocks per workgroup does not fit the LDS", kb_max);
  // more dynamic LDS than a kernel may use without asking: once per device
  static std::atomic<uint64_t> configured{0};
  if (int rc = allow_dynamic_lds(configured, reinterpret_cast<const void*>(&fp8_tile_kernel<TO, false, WM>), kLdsMax)) return rc;
  Fp8TileParams p{};
  p.a = q.a;
  p.a_s = q.a_s;
  p.b = q.b;
  p.b_s = q.b_s;
  p.out = q.out;
  p.out32 = q.out32;
  p.partial = partial;
  p.M = q.M;
  p.N = q.N;
  p.K = q.K;
  p.tiles_m = plan.tiles_m;
  p.tiles_n = plan.tiles_n;
  p.main_items = plan.main_items;
  p.splits = plan.splits;
  p.kb_per_split = plan.kt_per_split;
  p.as_row_bytes = 4;
  p.as_kb_bytes = 4 * q.M;
  fp8_tile_kernel<TO, false, WM><<<plan.grid, 512, lds, s>>>(p);
  if (plan.splits > 1) {
    const unsigned cut = plan.tiles_m * plan.tiles_n - plan.main_items;
    splitk_reduce_kernel<TO, 32 * WM><<<cut * (4 * WM), 256, 0, s>>>(partial, static_cast<uint16_t*>(p.out), p.M, p.N, p.tiles_m,
                                                                    p.tiles_n, p.main_items, p.splits, p.out32);
  }
  return KSQ_OK;
}

// grouped (MoE) form of the tile kernel: one 256-slot block of the aligned permutation per row tile
template <typename TO, int WM>
int launch_fp8_tile_grouped(const Fp8Params& q, unsigned blocks, hipStream_t s) {
  constexpr int kLdsMax = 160 * 1024;
  // (the 256-slot kernel runs half-empty blocks on the 128-token tile's three stages)
  const size_t lds = WM == 8 ? std::max(fp8_tile_lds_bytes(8, q.K / 128), fp8_tile_lds_bytes(4, q.K / 128))
                             : fp8_tile_lds_bytes(WM, q.K / 128);
  if (lds > kLdsMax) return fail(KSQ_ERR_UNSUPPORTED, "k range of %u blocks per workgroup does not fit the LDS", q.K / 128);
  // more dynamic LDS than a kernel may use without asking: once per device
  static std::atomic<uint64_t> configured{0};
  if (int rc = allow_dynamic_lds(configured, reinterpret_cast<const void*>(&fp8_tile_kernel<TO, true, WM>), kLdsMax)) return rc;
  Fp8TileParams p{};
  p.a = q.a;
  p.a_s = q.a_s;
  p.b = q.b;
  p.b_s = q.b_s;
  p.out = q.out;
  p.M = q.M;
  p.N = q.N;
  p.K = q.K;
  p.tiles_m = blocks;
  p.tiles_n = static_cast<uint32_t>(div_up(q.N, 256));
  p.main_items = 0;
  p.splits = 1;
  p.kb_per_split = q.K / 128;
  p.as_row_bytes = q.as_row_stride * 4;
  p.as_kb_bytes = q.as_kb_stride * 4;
  p.sorted_ids = q.sorted_ids;
  p.expert_ids = q.expert_ids;
  p.num_post_pad = q.num_post_pad;
  p.topk_w = q.topk_w;
  p.numel = q.numel;
  p.top_k = q.top_k;
  p.scale_rows = q.scale_rows;
  fp8_tile_kernel<TO, true, WM><<<p.tiles_m * p.tiles_n, 512, lds, s>>>(p);
  return KSQ_OK;
}

// per-tensor scales spread into the blockwise layouts
__global__ void __launch_bounds__(256) fp8_expand_scales_kernel(const float* __restrict__ a_scale, const float* __restrict__ b_scale,
                                                                float* __restrict__ a_s, size_t na, float* __restrict__ b_s,
                                                                size_t nb) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < na) a_s[i] = a_scale[0];
  if (i < nb) b_s[i] = b_scale[0];
}

inline size_t align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT size_t ksq_fp8_blockwise_workspace_size(size_t max_m, size_t n, size_t k) {
  // only the split-K form of the tile kernel needs scratch: fp32 partial tiles
  if (n == 0 || k == 0 || k % 128 != 0) return 0;
  size_t need = 0;
  // the plan is the same for all m of a band of 128 rows
  for (size_t band_end = 128; max_m > 32; band_end += 128) {
    const size_t m = band_end < max_m ? band_end : max_m;
    const TilePlan t = plan_fp8_tile(m, n, k);
    need = t.workspace_bytes > need ? t.workspace_bytes : need;
    if (m == max_m) break;
  }
  return need;
}

namespace {
// out32 given (verification entry point): the same kernels under the same plan, with the fp32 sums stored to out32
// [m, n] instead of rounded into out (which is then not touched)
int fp8_blockwise_gemm_impl(const char* fn, const void* a_q, const void* a_s, const void* b, const void* b_s, void* out,
                            size_t m, size_t n, size_t k, int out_dtype, void* workspace, size_t workspace_bytes,
                            void* stream, float* out32) {
  if (out32) out = out32;
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
  p.out32 = out32;
  p.as_row_stride = 1;
  p.as_kb_stride = static_cast<uint32_t>(m);
  int rc;
  if (use_fp8_tile(m, n, k)) {
    const TilePlan plan = plan_fp8_tile(m, n, k);
    if (plan.splits > 1 && (!workspace || workspace_bytes < plan.workspace_bytes || !aligned16(workspace)))
      return fail(KSQ_ERR_WORKSPACE, "%s: m=%zu n=%zu k=%zu needs %zu bytes of 16-byte aligned workspace, got %zu", fn, m,
                  n, k, plan.workspace_bytes, workspace ? workspace_bytes : size_t(0));
    if (256 * k > 0xffffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k too large", fn);
    float* partial = plan.splits > 1 ? static_cast<float*>(workspace) : nullptr;
    if (plan.block_m == 128)
      rc = out_dtype == KSQ_F16 ? launch_fp8_tile<F16, 4>(p, plan, partial, as_stream(stream))
                                : launch_fp8_tile<BF16, 4>(p, plan, partial, as_stream(stream));
    else
      rc = out_dtype == KSQ_F16 ? launch_fp8_tile<F16, 8>(p, plan, partial, as_stream(stream))
                                : launch_fp8_tile<BF16, 8>(p, plan, partial, as_stream(stream));
  } else {
    rc = out_dtype == KSQ_F16 ? dispatch<F16>(p, as_stream(stream)) : dispatch<BF16>(p, as_stream(stream));
  }
  if (rc) return rc;
  return check_launch(fn);
}
}  // namespace

KSQ_EXPORT int ksq_fp8_blockwise_gemm(const void* a_q, const void* a_s, const void* b, const void* b_s, void* out,
                                      size_t m, size_t n, size_t k, int out_dtype, void* workspace,
                                      size_t workspace_bytes, void* stream) {
  if (out_dtype == KSQ_F32)  // fp32 activations: the sums are the output (the reference instantiates InvokeBlockGemm<float>)
    return fp8_blockwise_gemm_impl("ksq_fp8_blockwise_gemm", a_q, a_s, b, b_s, nullptr, m, n, k, KSQ_BF16, workspace,
                                   workspace_bytes, stream, static_cast<float*>(out));
  return fp8_blockwise_gemm_impl("ksq_fp8_blockwise_gemm", a_q, a_s, b, b_s, out, m, n, k, out_dtype, workspace,
                                 workspace_bytes, stream, nullptr);
}

KSQ_EXPORT int ksq_fp8_blockwise_gemm_f32(const void* a_q, const void* a_s, const void* b, const void* b_s, float* out,
                                          size_t m, size_t n, size_t k, void* workspace, size_t workspace_bytes,
                                          void* stream) {
  return fp8_blockwise_gemm_impl("ksq_fp8_blockwise_gemm_f32", a_q, a_s, b, b_s, nullptr, m, n, k, KSQ_BF16, workspace,
                                 workspace_bytes, stream, out);
}

KSQ_EXPORT int ksq_moe_fp8_blockwise_gemm(void* out, const void* a_q, const void* a_s, int a_s_column_major, size_t a_rows, const void* b,
                                          const void* b_s, const void* topk_w, const void* sorted_ids,
                                          const void* expert_ids, const void* num_post_pad, size_t numel, size_t top_k,
                                          size_t E, size_t n, size_t k, size_t block_m, int out_dtype, void* stream) {
  const char* fn = "ksq_moe_fp8_blockwise_gemm";
  if (!a_q || !a_s || !b || !b_s || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  // sorted_ids == NULL: a handful of slots, one per 16-row block, with the router's ids in expert_ids
  const bool few = !sorted_ids;
  if (!expert_ids || (!few && !num_post_pad)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null index buffer", fn);
  if (few && (block_m != 16 || numel > 64))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: without sorted_ids every slot is a 16-row block of its own: block_m 16, at most 64 slots", fn);
  if (!aligned16(a_q) || !aligned16(b) || !aligned16(out) || (reinterpret_cast<uintptr_t>(a_s) & 3u) ||
      (reinterpret_cast<uintptr_t>(b_s) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: a_q, b, out must be 16-byte aligned, scales 4-byte aligned", fn);
  if (n == 0 || k == 0 || k % 128 != 0 || n % 16 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need k %% 128 == 0 and n %% 16 == 0 (n=%zu k=%zu)", fn, n, k);
  if (out_dtype != KSQ_F16 && out_dtype != KSQ_BF16)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: output dtype must be f16 or bf16", fn);
  if (top_k == 0 || E == 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: top_k and E must be positive", fn);
  if (block_m != 16 && block_m != 32 && block_m != 128 && block_m != 256)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: block_m %zu not in {16,32,128,256}", fn, block_m);
  if (numel == 0) return KSQ_OK;
  if (a_rows < (numel + top_k - 1) / top_k)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: %zu activation rows cannot serve %zu slots of top_k %zu", fn, a_rows, numel, top_k);
  if (numel > 0x7fffffffull || a_rows > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: dimension too large", fn);
  const size_t cap_blocks = few ? numel : (numel + E * (block_m - 1)) / block_m;  // upper bound on aligned blocks
  if (cap_blocks > 65535) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: too many row blocks (%zu)", fn, cap_blocks);
  Fp8Params p{static_cast<const uint8_t*>(a_q), static_cast<const float*>(a_s), static_cast<const uint8_t*>(b),
              static_cast<const float*>(b_s), out, static_cast<uint32_t>(cap_blocks * block_m), static_cast<uint32_t>(n),
              static_cast<uint32_t>(k)};
  p.as_row_stride = a_s_column_major ? 1u : static_cast<uint32_t>(k / 128);
  p.as_kb_stride = a_s_column_major ? static_cast<uint32_t>(a_rows) : 1u;
  p.sorted_ids = static_cast<const int32_t*>(sorted_ids);
  p.expert_ids = static_cast<const int32_t*>(expert_ids);
  p.num_post_pad = static_cast<const int32_t*>(num_post_pad);
  p.topk_w = static_cast<const float*>(topk_w);
  p.numel = static_cast<uint32_t>(numel);
  p.top_k = static_cast<uint32_t>(top_k);
  p.scale_rows = static_cast<uint32_t>(div_up(n, 128));
  p.num_experts = static_cast<uint32_t>(E);
  const int mt = block_m == 16 ? 1 : 2;
  const unsigned blocks = static_cast<unsigned>(cap_blocks);
  int rc;
  if (block_m >= 128) {  // prefill regime: MFMA tile kernel, rows gathered / scattered through the permutation
    if (a_rows * k > 0xffffffffull || a_rows * (k / 128) * 4 > 0xffffffffull)
      return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: activations too large", fn);
    if (block_m == 128)
      rc = out_dtype == KSQ_F16 ? launch_fp8_tile_grouped<F16, 4>(p, blocks, as_stream(stream))
                                : launch_fp8_tile_grouped<BF16, 4>(p, blocks, as_stream(stream));
    else
      rc = out_dtype == KSQ_F16 ? launch_fp8_tile_grouped<F16, 8>(p, blocks, as_stream(stream))
                                : launch_fp8_tile_grouped<BF16, 8>(p, blocks, as_stream(stream));
  } else {
    rc = out_dtype == KSQ_F16 ? dispatch_grouped<F16>(p, mt, blocks, as_stream(stream))
                              : dispatch_grouped<BF16>(p, mt, blocks, as_stream(stream));
  }
  if (rc) return rc;
  return check_launch(fn);
}

KSQ_EXPORT int ksq_moe_fp8_down_sum(void* out, const void* a_q, const void* a_s, const void* b, const void* b_s,
                                    const void* topk_w, const void* topk_ids, size_t tokens, size_t top_k, size_t E, size_t n,
                                    size_t k, int out_dtype, void* stream) {
  const char* fn = "ksq_moe_fp8_down_sum";
  if (!a_q || !a_s || !b || !b_s || !out || !topk_ids) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (!aligned16(a_q) || !aligned16(b) || !aligned16(out) || (reinterpret_cast<uintptr_t>(a_s) & 3u) ||
      (reinterpret_cast<uintptr_t>(b_s) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: a_q, b, out must be 16-byte aligned, scales 4-byte aligned", fn);
  if (n == 0 || k == 0 || k % 128 != 0 || n % 16 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need k %% 128 == 0 and n %% 16 == 0 (n=%zu k=%zu)", fn, n, k);
  if (out_dtype != KSQ_F16 && out_dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: output dtype must be f16 or bf16", fn);
  if (top_k == 0 || top_k > 32 || E == 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: top_k must be in 1..32 and E positive", fn);
  if (tokens == 0) return KSQ_OK;
  if (tokens > 8) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: at most 8 tokens (every token streams its own experts)", fn);
  if (n > 0x7fffffffull || top_k * k > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: dimension too large", fn);
  Fp8Params p{static_cast<const uint8_t*>(a_q), static_cast<const float*>(a_s), static_cast<const uint8_t*>(b),
              static_cast<const float*>(b_s), out, static_cast<uint32_t>(tokens), static_cast<uint32_t>(n),
              static_cast<uint32_t>(top_k * k)};  // a token's top_k rows of a, one behind the other
  p.kb_per_expert = static_cast<uint32_t>(k / 128);
  p.as_row_stride = static_cast<uint32_t>(top_k * (k / 128));  // scales [numel, k/128] row-major: a token's run on
  p.as_kb_stride = 1;
  p.expert_ids = static_cast<const int32_t*>(topk_ids);
  p.topk_w = static_cast<const float*>(topk_w);
  p.numel = static_cast<uint32_t>(tokens);  // rows of the output
  p.top_k = static_cast<uint32_t>(top_k);
  p.num_experts = static_cast<uint32_t>(E);
  p.scale_rows = static_cast<uint32_t>(div_up(n, 128));
  const bool four = n % 64 == 0 && (n / 64) * tokens >= 192;
  dim3 grid(static_cast<unsigned>(n / (four ? 64 : (n % 32 == 0 ? 32 : 16))), static_cast<unsigned>(tokens), 1);
  hipStream_t st = as_stream(stream);
#define KSQ_TOKSUM(TO_, NT_) fp8_splitk_kernel<TO_, 1, NT_, 4, 2, true, true><<<grid, 4 * 64, 0, st>>>(p)
  if (out_dtype == KSQ_F16) {
    if (four) KSQ_TOKSUM(F16, 4); else if (n % 32 == 0) KSQ_TOKSUM(F16, 2); else KSQ_TOKSUM(F16, 1);
  } else {
    if (four) KSQ_TOKSUM(BF16, 4); else if (n % 32 == 0) KSQ_TOKSUM(BF16, 2); else KSQ_TOKSUM(BF16, 1);
  }
#undef KSQ_TOKSUM
  return check_launch(fn);
}

KSQ_EXPORT size_t ksq_fp8_tensor_gemm_workspace_size(size_t max_m, size_t n, size_t k) {
  if (n == 0 || k == 0 || k % 128 != 0) return 0;
  return align256(max_m * (k / 128) * sizeof(float)) + align256(div_up(n, 128) * (k / 128) * sizeof(float)) +
         ksq_fp8_blockwise_workspace_size(max_m, n, k);
}

KSQ_EXPORT int ksq_fp8_tensor_gemm(const void* a_q, const void* a_scale, const void* b, const void* b_scale, void* out,
                                   size_t m, size_t n, size_t k, int out_dtype, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  const char* fn = "ksq_fp8_tensor_gemm";
  if (!a_q || !a_scale || !b || !b_scale || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if ((reinterpret_cast<uintptr_t>(a_scale) & 3u) || (reinterpret_cast<uintptr_t>(b_scale) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: scales must be 4-byte aligned", fn);
  if (n == 0 || k == 0 || k % 128 != 0 || n % 16 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need k %% 128 == 0 and n %% 16 == 0 (n=%zu k=%zu)", fn, n, k);
  if (m == 0) return KSQ_OK;
  const size_t kb = k / 128;
  const size_t na = m * kb, nb = div_up(n, 128) * kb;
  const size_t a_bytes = align256(na * sizeof(float)), b_bytes = align256(nb * sizeof(float));
  const size_t need = a_bytes + b_bytes + ksq_fp8_blockwise_workspace_size(m, n, k);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return fail(KSQ_ERR_WORKSPACE, "%s: m=%zu n=%zu k=%zu needs %zu bytes of 256-byte aligned workspace, got %zu", fn, m, n, k,
                need, workspace ? workspace_bytes : size_t(0));
  char* ws = static_cast<char*>(workspace);
  float* a_s = reinterpret_cast<float*>(ws);
  float* b_s = reinterpret_cast<float*>(ws + a_bytes);
  const size_t most = na > nb ? na : nb;
  fp8_expand_scales_kernel<<<static_cast<unsigned>(div_up(most, 256)), 256, 0, as_stream(stream)>>>(
      static_cast<const float*>(a_scale), static_cast<const float*>(b_scale), a_s, na, b_s, nb);
  return ksq_fp8_blockwise_gemm(a_q, a_s, b, b_s, out, m, n, k, out_dtype, ws + a_bytes + b_bytes,
                                workspace_bytes - a_bytes - b_bytes, stream);
}
