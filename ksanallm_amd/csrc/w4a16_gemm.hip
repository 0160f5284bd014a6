// ksq_w4a16_gemm / ksq_moe_w4a16_gemm: argument checks and kernel dispatch.
#include <algorithm>
#include <cstdlib>

#include "ksq_common.h"
#include <atomic>

#include "tile_select.h"
#include "w4a16_splitk.h"
#include "w4a16_tile.h"

namespace ksq {
namespace {

template <typename T, int MT, int NT, int WAVES, int GROUP, bool HAS_ZP, bool GROUPED, int XC = 0>
int launch_splitk(const SplitKParams& p, uint32_t m_blocks, hipStream_t s) {
  const uint32_t parts = (GROUPED || !p.partial) ? 1u : static_cast<uint32_t>(div_up(p.K / 128, p.kt_per_part));
  dim3 grid(p.N / 16 / NT, m_blocks, parts);
  // ring depth in k-tiles and the wavefronts per SIMD the register budget is cut for
  // (32-row blocks with four column tiles: two k-tiles ahead in the dense form, 12.9 against 14.0 us at n = 14336,
  // k = 4096; the grouped form measured 4 % slower with it and keeps one)
  // (the forms that stage x through LDS keep one k-tile in flight per wavefront: twice the wavefronts instead)
  // (two row tiles, eight column tiles and zero points in the register form: a ring of two does not fit the registers)
  constexpr int LOOK = XC > 0 ? 1
                              : (GROUP != 128 ? 2
                                              : (MT == 1 ? (NT == 1 ? 4 : (NT == 2 ? 3 : 2))
                                                         : ((NT <= 2 || (!GROUPED && !(NT == 8 && HAS_ZP))) ? 2 : 1)));
  constexpr int OCC = XC > 0 ? ((MT == 1 && NT == 4) ? 4 : 2)
                             : ((GROUP == 128 && MT == 1 && NT == 1) ? 4 : ((GROUP == 128 && MT == 1 && NT == 2) ? 3 : 2));
  typedef SplitKLds<MT, NT, WAVES, XC> Lds;
  auto kernel = &w4a16_splitk_kernel<T, MT, NT, WAVES, LOOK, OCC, GROUP, HAS_ZP, GROUPED, XC>;
  if (Lds::kBytes > 65536) {
    static std::atomic<uint64_t> configured{0};
    if (int rc = allow_dynamic_lds(configured, reinterpret_cast<const void*>(kernel), Lds::kBytes)) return rc;
  }
  kernel<<<grid, WAVES * 64, Lds::kBytes, s>>>(p);
  return KSQ_OK;
}

template <typename T, int MT, int NT, int WAVES, bool GROUPED, int XC = 0>
int dispatch_group_zp(const SplitKParams& p, uint32_t m_blocks, size_t group, hipStream_t s) {
  const bool zp = p.zeros != nullptr;
  if (group == 128) {
    if (zp) {
      if constexpr (!GROUPED) return launch_splitk<T, MT, NT, WAVES, 128, true, GROUPED, XC>(p, m_blocks, s);
      else return fail(KSQ_ERR_UNSUPPORTED, "grouped W4A16 GEMM with zero points is not built");
    }
    return launch_splitk<T, MT, NT, WAVES, 128, false, GROUPED, XC>(p, m_blocks, s);
  }
  if constexpr (NT <= 2 && WAVES == 4 && !GROUPED && XC == 0) {
    if (group == 64) {
      return zp ? launch_splitk<T, MT, NT, 4, 64, true, false>(p, m_blocks, s)
                : launch_splitk<T, MT, NT, 4, 64, false, false>(p, m_blocks, s);
    }
    if (group == 32) {
      return zp ? launch_splitk<T, MT, NT, 4, 32, true, false>(p, m_blocks, s)
                : launch_splitk<T, MT, NT, 4, 32, false, false>(p, m_blocks, s);
    }
  }
  return fail(KSQ_ERR_UNSUPPORTED, "group size %zu has no kernel for this tile", group);
}

template <typename T, bool GROUPED>
int dispatch_tile(SplitKParams& p, SplitKChoice c, uint32_t m_blocks, size_t group, hipStream_t s) {
  if (group != 128) {  // small groups are only built for the narrow 4-wavefront shapes
    c.nt = (p.N / 16) % 2 == 0 ? 2 : 1;
    c.waves = 4;
    c.xc = 0;
  }
  p.nibble_mask = 0x000f000fu;
  p.magic2 = T::kMagic2;
  if (c.xc == 8 && c.mt == 1 && c.nt == 4 && c.waves == 8) return dispatch_group_zp<T, 1, 4, 8, GROUPED, 8>(p, m_blocks, group, s);
  if (c.xc == 8 && c.mt == 1 && c.nt == 8 && c.waves == 8) return dispatch_group_zp<T, 1, 8, 8, GROUPED, 8>(p, m_blocks, group, s);
  if (c.xc == 8 && c.mt == 2 && c.nt == 4 && c.waves == 8) return dispatch_group_zp<T, 2, 4, 8, GROUPED, 8>(p, m_blocks, group, s);
  if (c.xc == 4 && c.mt == 2 && c.nt == 8 && c.waves == 4) return dispatch_group_zp<T, 2, 8, 4, GROUPED, 4>(p, m_blocks, group, s);
  if (c.xc != 0) return fail(KSQ_ERR_UNSUPPORTED, "no split-K kernel for mt=%d nt=%d waves=%d xc=%d", c.mt, c.nt, c.waves, c.xc);
#define KSQ_CASE(MT_, NT_, W_)                                    \
  if (c.mt == MT_ && c.nt == NT_ && c.waves == W_)                \
    return dispatch_group_zp<T, MT_, NT_, W_, GROUPED>(p, m_blocks, group, s);
  KSQ_CASE(1, 8, 8)
  KSQ_CASE(1, 4, 8)
  KSQ_CASE(1, 2, 8)
  KSQ_CASE(1, 1, 8)
  KSQ_CASE(1, 8, 4)
  KSQ_CASE(1, 4, 4)
  KSQ_CASE(1, 2, 4)
  KSQ_CASE(1, 1, 4)
  KSQ_CASE(2, 4, 8)
  KSQ_CASE(2, 2, 8)
  KSQ_CASE(2, 1, 8)
  KSQ_CASE(2, 8, 4)
  KSQ_CASE(2, 4, 4)
  KSQ_CASE(2, 2, 4)
  KSQ_CASE(2, 1, 4)
#undef KSQ_CASE
  return fail(KSQ_ERR_UNSUPPORTED, "no split-K kernel for mt=%d nt=%d waves=%d", c.mt, c.nt, c.waves);
}

// Workspace of a decode launch that cuts K over `parts` workgroups: the fp32 partial sums [parts][m][n].
size_t splitk_workspace(const SplitKChoice& c, size_t m, size_t n) {
  return c.parts > 1 ? static_cast<size_t>(c.parts) * m * n * sizeof(float) : 0;
}

template <typename T, int WM, bool HAS_ZP, int GROUP>
int launch_tile_group(const TileParams& p, unsigned grid, hipStream_t s) {
  constexpr int kLds = 4 * WM * 2 * 1024;  // NS stages of WM*2 fragments
  // more dynamic LDS than a kernel may use without asking: once per device
  static std::atomic<uint64_t> configured{0};
  auto kernel = &w4a16_tile_kernel<T, WM, HAS_ZP, false, GROUP>;
  if (int rc = allow_dynamic_lds(configured, reinterpret_cast<const void*>(kernel), kLds)) return rc;
  kernel<<<grid, 512, kLds, s>>>(p);
  return KSQ_OK;
}

template <typename T, int WM, bool HAS_ZP>
int launch_tile_zp(const TileParams& p, unsigned grid, size_t group, hipStream_t s) {
  if (group == 64) return launch_tile_group<T, WM, HAS_ZP, 64>(p, grid, s);
  if (group == 32) return launch_tile_group<T, WM, HAS_ZP, 32>(p, grid, s);
  return launch_tile_group<T, WM, HAS_ZP, 128>(p, grid, s);
}

// grouped (MoE) form: one 128-row block of the aligned permutation per row tile, no split-K
template <typename T, int WM>
int launch_tile_grouped(const TileParams& p, hipStream_t s) {
  constexpr int kLds = 4 * WM * 2 * 1024;
  // more dynamic LDS than a kernel may use without asking: once per device
  static std::atomic<uint64_t> configured{0};
  if (int rc = allow_dynamic_lds(configured, reinterpret_cast<const void*>(&w4a16_tile_kernel<T, WM, false, true>), kLds)) return rc;
  w4a16_tile_kernel<T, WM, false, true><<<p.tiles_m * p.tiles_n, 512, kLds, s>>>(p);
  return KSQ_OK;
}

template <typename T>
int dispatch_mfma_tile(TileParams p, const TilePlan& plan, size_t group, hipStream_t s) {
  p.tiles_m = plan.tiles_m;
  p.tiles_n = plan.tiles_n;
  p.main_items = plan.main_items;
  p.splits = plan.splits;
  p.kt_per_split = plan.kt_per_split;
  int rc;
  if (plan.block_m == 128)
    rc = p.zeros ? launch_tile_zp<T, 8, true>(p, plan.grid, group, s) : launch_tile_zp<T, 8, false>(p, plan.grid, group, s);
  else
    rc = p.zeros ? launch_tile_zp<T, 16, true>(p, plan.grid, group, s) : launch_tile_zp<T, 16, false>(p, plan.grid, group, s);
  if (rc) return rc;
  if (plan.splits > 1) {
    const unsigned cut = plan.tiles_m * plan.tiles_n - plan.main_items;
    uint16_t* y = static_cast<uint16_t*>(p.y);
    if (plan.block_m == 128)
      splitk_reduce_kernel<T, 128><<<cut * 16, 256, 0, s>>>(p.partial, y, p.M, p.N, p.tiles_m, p.tiles_n, p.main_items, p.splits, p.y32);
    else
      splitk_reduce_kernel<T, 256><<<cut * 32, 256, 0, s>>>(p.partial, y, p.M, p.N, p.tiles_m, p.tiles_n, p.main_items, p.splits, p.y32);
  }
  return KSQ_OK;
}

int check_common(const char* fn, const void* y, const void* x, const void* w, const void* sc, size_t n, size_t k,
                 size_t group, int dtype) {
  if (!y || !x || !w || !sc) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (!aligned16(y) || !aligned16(x) || !aligned16(w) || !aligned16(sc))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
  if (n == 0 || k == 0 || k % 128 != 0 || n % 16 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need k %% 128 == 0 and n %% 16 == 0 (n=%zu k=%zu)", fn, n, k);
  if (group != 32 && group != 64 && group != 128)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: group size %zu not in {32,64,128}", fn, group);
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  if (n > 0x7fffffffull || k > 0x7fffffffull || k / 128 * 1024 * 8 > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: dimension too large", fn);
  return KSQ_OK;
}

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT size_t ksq_w4a16_workspace_size(size_t max_m, size_t n, size_t k, size_t group, int dtype) {
  (void)dtype;
  // fp32 partials: the decode kernel when it cuts K over workgroups, the tile kernel for the tiles it cuts along K
  if (n == 0 || k == 0 || k % 128 != 0) return 0;
  size_t need = 0;
  // decode kernel: partial sums when K is cut over workgroups
  if (group == 128) {
    for (size_t m = 1; m <= max_m && m <= kRowBlockMaxM; ++m) {
      if (m > 32 && !small_w4a16_problem(m, n, k, group)) break;  // (monotonic in m: no decode-form call above this m)
      const size_t bytes = splitk_workspace(select_splitk(m, n, k), m, n);
      need = bytes > need ? bytes : need;
    }
  }
  // the plan is the same for all m of a band of 128 rows
  for (size_t band_end = 128; max_m > 32; band_end += 128) {
    const size_t m = band_end < max_m ? band_end : max_m;
    if (group == 128 || group == 64 || group == 32) {  // (whether or not the small-problem rule sends this m elsewhere)
      const TilePlan t = plan_mfma_tile(m, n, k);
      need = t.workspace_bytes > need ? t.workspace_bytes : need;
    }
    if (m == max_m) break;
  }
  return need;
}

namespace {
// y32 given (verification entry point): the same kernels under the same plan, with the fp32 sums stored to y32 [m, n]
// instead of rounded to T into y (which is then not touched and may be null)
int w4a16_gemm_impl(const char* fn, void* y, const void* x, const void* w_packed, const void* scales_packed,
                    const void* zeros_packed, void* workspace, size_t workspace_bytes, size_t m, size_t n, size_t k,
                    size_t group, int dtype, void* stream, float* y32 = nullptr) {
  if (int rc = check_common(fn, y32 ? static_cast<void*>(y32) : y, x, w_packed, scales_packed, n, k, group, dtype)) return rc;
  if (m == 0) return KSQ_OK;
  if (m > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: m too large", fn);
  if (!use_mfma_tile(m, n, k, group) && m * k * 2 >= 0x40000000ull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: m too large for this shape", fn);
  SplitKParams p{};
  p.y = y;
  p.x = x;
  p.w = w_packed;
  p.scales = scales_packed;
  p.zeros = zeros_packed;
  p.M = static_cast<uint32_t>(m);
  p.N = static_cast<uint32_t>(n);
  p.K = static_cast<uint32_t>(k);
  p.x_bytes = static_cast<uint32_t>(m * k * 2);
  if (use_mfma_tile(m, n, k, group)) {
    TileParams tp{};
    tp.y = y;
    tp.x = x;
    tp.w = w_packed;
    tp.scales = scales_packed;
    tp.zeros = zeros_packed;
    tp.M = static_cast<uint32_t>(m);
    tp.N = static_cast<uint32_t>(n);
    tp.K = static_cast<uint32_t>(k);
    tp.y32 = y32;
    const TilePlan plan = plan_mfma_tile(m, n, k);
    if (plan.splits > 1) {
      if (!workspace || workspace_bytes < plan.workspace_bytes || !aligned16(workspace))
        return fail(KSQ_ERR_WORKSPACE, "%s: m=%zu n=%zu k=%zu needs %zu bytes of 16-byte aligned workspace, got %zu", fn,
                    m, n, k, plan.workspace_bytes, workspace ? workspace_bytes : size_t(0));
      tp.partial = static_cast<float*>(workspace);
    }
    if (256 * k * 2 > 0xffffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k too large", fn);
    int rc = dtype == KSQ_F16 ? dispatch_mfma_tile<F16>(tp, plan, group, as_stream(stream))
                              : dispatch_mfma_tile<BF16>(tp, plan, group, as_stream(stream));
    if (rc) return rc;
    return check_launch(fn);
  }
  SplitKChoice c = select_splitk(m, n, k);
  const size_t m_blocks = div_up(m, 16 * c.mt);
  if (m_blocks > 65535) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: m too large for the decode kernel", fn);
  p.partial = nullptr;
  p.kt_per_part = static_cast<uint32_t>(k / 128);
  if (c.parts > 1 && group == 128) {
    const size_t need = splitk_workspace(c, m, n);
    if (!workspace || workspace_bytes < need || !aligned16(workspace))
      return fail(KSQ_ERR_WORKSPACE, "%s: m=%zu n=%zu k=%zu needs %zu bytes of 16-byte aligned workspace, got %zu", fn, m, n,
                  k, need, workspace ? workspace_bytes : size_t(0));
    p.partial = static_cast<float*>(workspace);
    p.kt_per_part = static_cast<uint32_t>(div_up(k / 128, c.parts));
  }
  const bool one_part_f32 = y32 && !p.partial;  // the kernel's partial-sum store with a single part is the fp32 output
  if (one_part_f32) p.partial = y32;
  int rc = dtype == KSQ_F16 ? dispatch_tile<F16, false>(p, c, static_cast<uint32_t>(m_blocks), group, as_stream(stream))
                            : dispatch_tile<BF16, false>(p, c, static_cast<uint32_t>(m_blocks), group, as_stream(stream));
  if (rc) return rc;
  if (p.partial && !one_part_f32) {
    const size_t mn = m * n;
    const uint32_t parts = static_cast<uint32_t>(div_up(k / 128, p.kt_per_part));
    const unsigned blocks = static_cast<unsigned>(div_up(mn, 256 * 4));
    if (dtype == KSQ_F16)
      parts_reduce_kernel<F16><<<blocks, 256, 0, as_stream(stream)>>>(p.partial, static_cast<uint16_t*>(y), mn, parts, y32);
    else
      parts_reduce_kernel<BF16><<<blocks, 256, 0, as_stream(stream)>>>(p.partial, static_cast<uint16_t*>(y), mn, parts, y32);
  }
  return check_launch(fn);
}
}  // namespace

KSQ_EXPORT int ksq_w4a16_gemm(void* y, const void* x, const void* w_packed, const void* scales_packed,
                              const void* zeros_packed, void* workspace, size_t workspace_bytes, size_t m, size_t n,
                              size_t k, size_t group, int dtype, void* stream) {
  return w4a16_gemm_impl("ksq_w4a16_gemm", y, x, w_packed, scales_packed, zeros_packed, workspace, workspace_bytes, m, n, k,
                         group, dtype, stream);
}

KSQ_EXPORT int ksq_w4a16_gemm_f32(float* y, const void* x, const void* w_packed, const void* scales_packed,
                                  const void* zeros_packed, void* workspace, size_t workspace_bytes, size_t m, size_t n,
                                  size_t k, size_t group, int dtype, void* stream) {
  return w4a16_gemm_impl("ksq_w4a16_gemm_f32", nullptr, x, w_packed, scales_packed, zeros_packed, workspace, workspace_bytes, m,
                         n, k, group, dtype, stream, y);
}

namespace {
template <typename T, int NT>
int launch_token_sum(const SplitKParams& p, uint32_t tokens, hipStream_t s) {
  // one row of x per workgroup: the narrow decode instances' ring depths
  constexpr int LOOK = NT == 1 ? 4 : 3, OCC = NT == 1 ? 4 : 3;
  typedef SplitKLds<1, NT, 4, 0> Lds;
  dim3 grid(p.N / 16 / NT, tokens, 1);
  w4a16_splitk_kernel<T, 1, NT, 4, LOOK, OCC, 128, false, true, 0, 16, true><<<grid, 4 * 64, Lds::kBytes, s>>>(p);
  return KSQ_OK;
}
}  // namespace

KSQ_EXPORT int ksq_moe_w4a16_down_sum(void* out, const void* x, const void* w_packed, const void* scales_packed,
                                      const void* topk_w, const void* topk_ids, size_t tokens, size_t top_k, size_t E,
                                      size_t n, size_t k, size_t group, int dtype, void* stream) {
  const char* fn = "ksq_moe_w4a16_down_sum";
  if (int rc = check_common(fn, out, x, w_packed, scales_packed, n, k, group, dtype)) return rc;
  if (!topk_ids) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null index buffer", fn);
  if (group != 128) return fail(KSQ_ERR_UNSUPPORTED, "%s: expert weights need group size 128", fn);
  if (top_k == 0 || top_k > 32 || E == 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: top_k must be in 1..32 and E positive", fn);
  if (tokens == 0) return KSQ_OK;
  if (tokens > 8) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: at most 8 tokens (every token streams its own experts)", fn);
  if (tokens * top_k * k * 2 >= 0x40000000ull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: x too large", fn);
  SplitKParams p{};
  p.y = out;
  p.x = x;
  p.w = w_packed;
  p.scales = scales_packed;
  p.M = static_cast<uint32_t>(tokens);
  p.N = static_cast<uint32_t>(n);
  p.K = static_cast<uint32_t>(top_k * k);  // a token's top_k rows of x, one behind the other
  p.kt_per_expert = static_cast<uint32_t>(k / 128);
  p.expert_ids = static_cast<const int32_t*>(topk_ids);
  p.topk_w = static_cast<const float*>(topk_w);
  p.numel = static_cast<uint32_t>(tokens);  // rows of the output
  p.top_k = static_cast<uint32_t>(top_k);
  p.num_experts = static_cast<uint32_t>(E);
  p.x_bytes = static_cast<uint32_t>(tokens * top_k * k * 2);
  p.nibble_mask = 0x000f000fu;
  // two column tiles per workgroup where that still leaves a workgroup for most CUs
  const bool two = (n / 16) % 2 == 0 && (n / 32) * tokens >= 192;
  p.magic2 = dtype == KSQ_F16 ? F16::kMagic2 : BF16::kMagic2;
  int rc;
  if (dtype == KSQ_F16)
    rc = two ? launch_token_sum<F16, 2>(p, static_cast<uint32_t>(tokens), as_stream(stream))
             : launch_token_sum<F16, 1>(p, static_cast<uint32_t>(tokens), as_stream(stream));
  else
    rc = two ? launch_token_sum<BF16, 2>(p, static_cast<uint32_t>(tokens), as_stream(stream))
             : launch_token_sum<BF16, 1>(p, static_cast<uint32_t>(tokens), as_stream(stream));
  if (rc) return rc;
  return check_launch(fn);
}

// ---- the same GEMM for callers that cannot hand over a workspace --------------------------------------------------
// The fp32 partial sums of launches that cut K go through this array instead of a caller's buffer.  Every GPU the
// library runs on holds its own copy from the moment the code object is loaded until the process ends.  The name below is
// a host-side handle, not a device address: the address on the current device comes from hipGetSymbolAddress, once per
// device, and only that pointer is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[KSQ_W4A16_STATIC_WORKSPACE_BYTES];

namespace {
// device address of `scratch` on the current device (nullptr after recording the error)
void* static_scratch() {
  static std::atomic<void*> addr[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    set_error("ksq_w4a16_gemm_static: cannot tell the current device");
    return nullptr;
  }
  void* p = addr[dev].load(std::memory_order_acquire);
  if (p) return p;
  const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p) {
    set_error("ksq_w4a16_gemm_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    return nullptr;
  }
  addr[dev].store(p, std::memory_order_release);  // every thread that races here stores the same address
  return p;
}
}  // namespace

KSQ_EXPORT size_t ksq_w4a16_static_workspace_bytes(void) { return KSQ_W4A16_STATIC_WORKSPACE_BYTES; }

KSQ_EXPORT int ksq_w4a16_gemm_static(void* y, const void* x, const void* w_packed, const void* scales_packed,
                                     const void* zeros_packed, size_t m, size_t n, size_t k, size_t group, int dtype,
                                     void* stream) {
  const char* fn = "ksq_w4a16_gemm_static";
  // what this very call needs (the plan of its m, not the maximum over a range of m)
  size_t need = 0;
  if (m > 0 && n > 0 && k > 0 && k % 128 == 0 && n % 16 == 0) {
    if (use_mfma_tile(m, n, k, group))
      need = plan_mfma_tile(m, n, k).workspace_bytes;
    else if (group == 128)
      need = splitk_workspace(select_splitk(m, n, k), m, n);
  }
  if (need > KSQ_W4A16_STATIC_WORKSPACE_BYTES)
    return fail(KSQ_ERR_WORKSPACE, "%s: m=%zu n=%zu k=%zu needs %zu bytes of scratch, the built-in buffer holds %zu: call "
                "ksq_w4a16_gemm with a workspace", fn, m, n, k, need, size_t(KSQ_W4A16_STATIC_WORKSPACE_BYTES));
  void* ws = nullptr;
  if (need > 0) {
    ws = static_scratch();
    if (!ws) return KSQ_ERR_LAUNCH;
  }
  return w4a16_gemm_impl(fn, y, x, w_packed, scales_packed, zeros_packed, ws, need > 0 ? KSQ_W4A16_STATIC_WORKSPACE_BYTES : 0,
                         m, n, k, group, dtype, stream);
}

namespace {
int moe_w4a16_gemm_impl(const char* fn, bool fuse_silu, void* out, const void* x, const void* w_packed,
                        const void* scales_packed, const void* zeros_packed, const void* topk_w, const void* sorted_ids,
                        const void* expert_ids, const void* num_post_pad, size_t numel, size_t top_k, size_t E, size_t n,
                        size_t k, size_t group, size_t block_m, int dtype, void* stream) {
  if (int rc = check_common(fn, out, x, w_packed, scales_packed, n, k, group, dtype)) return rc;
  if (fuse_silu) {
    if (n % 32 != 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: n = 2 * inter must be a multiple of 32", fn);
  }
  // sorted_ids == NULL: a handful of slots, one per 16-row block, with the router's ids in expert_ids (w4a16_splitk.h)
  const bool few = !sorted_ids;
  if (!expert_ids || (!few && !num_post_pad)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null index buffer", fn);
  if (few && (block_m != 16 || numel > 64))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: without sorted_ids every slot is a 16-row block of its own: block_m 16, at most 64 slots", fn);
  if (zeros_packed) return fail(KSQ_ERR_UNSUPPORTED, "%s: zero points are not supported for expert weights", fn);
  if (group != 128) return fail(KSQ_ERR_UNSUPPORTED, "%s: expert weights need group size 128", fn);
  if (top_k == 0 || E == 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: top_k and E must be positive", fn);
  if (block_m != 16 && block_m != 32 && block_m != 128 && block_m != 256)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: block_m %zu not in {16,32,128,256}", fn, block_m);
  if (numel == 0) return KSQ_OK;
  const size_t cap_blocks = few ? numel : (numel + E * (block_m - 1)) / block_m;  // upper bound on aligned blocks
  if (block_m >= 128) {  // prefill regime: MFMA tile kernel, rows gathered / scattered through the permutation
    if (numel > 0x7fffffffull || (numel / top_k + 1) * k * 2 > 0xffffffffull)
      return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: x too large", fn);
    TileParams tp{};
    tp.y = out;
    tp.x = x;
    tp.w = w_packed;
    tp.scales = scales_packed;
    tp.M = static_cast<uint32_t>(cap_blocks * block_m);
    tp.N = static_cast<uint32_t>(n);
    tp.K = static_cast<uint32_t>(k);
    tp.tiles_m = static_cast<uint32_t>(cap_blocks);
    tp.tiles_n = static_cast<uint32_t>(div_up(n, 256));  // paired: 128 gate + 128 up columns per workgroup, the same count
    tp.pair_tiles = fuse_silu ? static_cast<uint32_t>(n / 32) : 0;
    tp.main_items = 0;
    tp.splits = 1;
    tp.kt_per_split = static_cast<uint32_t>(k / 128);
    tp.sorted_ids = static_cast<const int32_t*>(sorted_ids);
    tp.expert_ids = static_cast<const int32_t*>(expert_ids);
    tp.num_post_pad = static_cast<const int32_t*>(num_post_pad);
    tp.topk_w = static_cast<const float*>(topk_w);
    tp.numel = static_cast<uint32_t>(numel);
    tp.top_k = static_cast<uint32_t>(top_k);
    int rc;
    if (block_m == 256)
      rc = dtype == KSQ_F16 ? launch_tile_grouped<F16, 16>(tp, as_stream(stream)) : launch_tile_grouped<BF16, 16>(tp, as_stream(stream));
    else
      rc = dtype == KSQ_F16 ? launch_tile_grouped<F16, 8>(tp, as_stream(stream)) : launch_tile_grouped<BF16, 8>(tp, as_stream(stream));
    if (rc) return rc;
    return check_launch(fn);
  }
  if (cap_blocks > 65535) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: too many row blocks (%zu)", fn, cap_blocks);
  const size_t x_rows = (numel + top_k - 1) / top_k;
  if (x_rows * k * 2 >= 0x40000000ull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: x too large", fn);
  SplitKParams p{};
  p.y = out;
  p.x = x;
  p.w = w_packed;
  p.scales = scales_packed;
  p.zeros = nullptr;
  p.M = static_cast<uint32_t>(cap_blocks);
  p.N = static_cast<uint32_t>(n);
  p.K = static_cast<uint32_t>(k);
  p.sorted_ids = static_cast<const int32_t*>(sorted_ids);
  p.expert_ids = static_cast<const int32_t*>(expert_ids);
  p.num_post_pad = static_cast<const int32_t*>(num_post_pad);
  p.topk_w = static_cast<const float*>(topk_w);
  p.numel = static_cast<uint32_t>(numel);
  p.top_k = static_cast<uint32_t>(top_k);
  p.num_experts = static_cast<uint32_t>(E);
  p.x_bytes = static_cast<uint32_t>(x_rows * k * 2);
  // about numel/block_m + E/2 of the aligned blocks hold rows; K is never split across workgroups here
  SplitKChoice c = select_splitk_blocks(static_cast<int>(block_m / 16),
                                        few ? numel : std::min(cap_blocks, numel / block_m + E / 2 + 1), n, k);
  if (fuse_silu) {
    if (c.nt < 2) c.nt = 2;  // a workgroup holds gate and up tiles in pairs
    p.pair_tiles = static_cast<uint32_t>(n / 32);
  }
  // activations through LDS (w4a16_splitk.h) as in the dense form: 2-3 % at E = 256, hidden 7168, inter 2048 from a
  // few tokens per expert on (64 tokens 813 -> 788 us, 512 tokens 1353 -> 1316 us for the whole block), not for a
  // handful of blocks (1 token: 50.1 -> 52.6 us)
  if ((n / 16) % 4 == 0 && numel >= 32) {
    if (c.mt == 2 && c.nt == 8) {
      c.waves = 4;
      c.xc = 4;
    } else if (c.mt == 2 && c.nt == 4) {
      c.waves = 8;
      c.xc = 8;
    } else if (c.mt == 1 && c.nt >= 4) {
      c.waves = 8;
      c.xc = 8;
    }
  }
  int rc = dtype == KSQ_F16 ? dispatch_tile<F16, true>(p, c, static_cast<uint32_t>(cap_blocks), group, as_stream(stream))
                            : dispatch_tile<BF16, true>(p, c, static_cast<uint32_t>(cap_blocks), group, as_stream(stream));
  if (rc) return rc;
  return check_launch(fn);
}
}  // namespace

KSQ_EXPORT int ksq_moe_w4a16_gemm(void* out, const void* x, const void* w_packed, const void* scales_packed,
                                  const void* zeros_packed, const void* topk_w, const void* sorted_ids,
                                  const void* expert_ids, const void* num_post_pad, size_t numel, size_t top_k,
                                  size_t E, size_t n, size_t k, size_t group, size_t block_m, int dtype,
                                  void* stream) {
  return moe_w4a16_gemm_impl("ksq_moe_w4a16_gemm", false, out, x, w_packed, scales_packed, zeros_packed, topk_w, sorted_ids,
                             expert_ids, num_post_pad, numel, top_k, E, n, k, group, block_m, dtype, stream);
}

KSQ_EXPORT int ksq_moe_w4a16_gate_up_silu(void* out, const void* x, const void* w_packed, const void* scales_packed,
                                          const void* zeros_packed, const void* sorted_ids, const void* expert_ids,
                                          const void* num_post_pad, size_t numel, size_t top_k, size_t E, size_t n,
                                          size_t k, size_t group, size_t block_m, int dtype, void* stream) {
  return moe_w4a16_gemm_impl("ksq_moe_w4a16_gate_up_silu", true, out, x, w_packed, scales_packed, zeros_packed, nullptr,
                             sorted_ids, expert_ids, num_post_pad, numel, top_k, E, n, k, group, block_m, dtype, stream);
}
