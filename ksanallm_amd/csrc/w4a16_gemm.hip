// ksq_w4a16_gemm / ksq_moe_w4a16_gemm: argument checks and kernel dispatch.
#include "ksq_common.h"
#include "tile_select.h"
#include "w4a16_splitk.h"

namespace ksq {
namespace {

template <typename T, int MT, int NT, int WAVES, int GROUP, bool HAS_ZP, bool GROUPED>
void launch_splitk(const SplitKParams& p, uint32_t m_blocks, hipStream_t s) {
  dim3 grid(p.N / 16 / NT, m_blocks, 1);
  w4a16_splitk_kernel<T, MT, NT, WAVES, GROUP, HAS_ZP, GROUPED><<<grid, WAVES * 64, 0, s>>>(p);
}

template <typename T, int MT, int NT, int WAVES, bool GROUPED>
int dispatch_group_zp(const SplitKParams& p, uint32_t m_blocks, size_t group, hipStream_t s) {
  const bool zp = p.zeros != nullptr;
  if (group == 128) {
    if (zp) {
      if constexpr (!GROUPED) launch_splitk<T, MT, NT, WAVES, 128, true, GROUPED>(p, m_blocks, s);
      else return fail(KSQ_ERR_UNSUPPORTED, "grouped W4A16 GEMM with zero points is not built");
    } else {
      launch_splitk<T, MT, NT, WAVES, 128, false, GROUPED>(p, m_blocks, s);
    }
    return KSQ_OK;
  }
  if constexpr (NT == 1 && WAVES == 8 && !GROUPED) {
    if (group == 64) {
      if (zp) launch_splitk<T, MT, 1, 8, 64, true, false>(p, m_blocks, s);
      else launch_splitk<T, MT, 1, 8, 64, false, false>(p, m_blocks, s);
      return KSQ_OK;
    }
    if (group == 32) {
      if (zp) launch_splitk<T, MT, 1, 8, 32, true, false>(p, m_blocks, s);
      else launch_splitk<T, MT, 1, 8, 32, false, false>(p, m_blocks, s);
      return KSQ_OK;
    }
  }
  return fail(KSQ_ERR_UNSUPPORTED, "group size %zu has no kernel for this tile", group);
}

template <typename T, bool GROUPED>
int dispatch_tile(const SplitKParams& p, SplitKChoice c, size_t group, hipStream_t s) {
  if (group != 128) {  // small groups are only built for the 1-tile, 8-wavefront shape
    c.nt = 1;
    c.waves = 8;
  }
  if (GROUPED) c.waves = 8;
  const uint32_t rows = GROUPED ? 0 : p.M;
  auto mb = [&](int mt) { return static_cast<uint32_t>(div_up(rows, 16 * mt)); };
  // grouped launches pass the number of blocks in p.M
  auto blocks = [&](int mt) { return GROUPED ? p.M : mb(mt); };
#define KSQ_CASE(MT_, NT_, W_)                                    \
  if (c.mt == MT_ && c.nt == NT_ && c.waves == W_)                \
    return dispatch_group_zp<T, MT_, NT_, W_, GROUPED>(p, blocks(MT_), group, s);
  KSQ_CASE(1, 1, 8)
  KSQ_CASE(2, 1, 8)
  KSQ_CASE(1, 2, 8)
  KSQ_CASE(2, 2, 8)
  if constexpr (!GROUPED) {
    KSQ_CASE(1, 1, 16)
    KSQ_CASE(2, 1, 16)
    KSQ_CASE(1, 2, 16)
    KSQ_CASE(2, 2, 16)
  }
#undef KSQ_CASE
  return fail(KSQ_ERR_UNSUPPORTED, "no split-K kernel for mt=%d nt=%d waves=%d", c.mt, c.nt, c.waves);
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
  if (n > 0x7fffffffull || k > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: dimension too large", fn);
  return KSQ_OK;
}

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT size_t ksq_w4a16_workspace_size(size_t max_m, size_t n, size_t k, size_t group, int dtype) {
  (void)max_m; (void)n; (void)k; (void)group; (void)dtype;
  return 0;  // every reduction happens inside a workgroup
}

KSQ_EXPORT int ksq_w4a16_gemm(void* y, const void* x, const void* w_packed, const void* scales_packed,
                              const void* zeros_packed, void* workspace, size_t workspace_bytes, size_t m, size_t n,
                              size_t k, size_t group, int dtype, void* stream) {
  const char* fn = "ksq_w4a16_gemm";
  (void)workspace; (void)workspace_bytes;
  if (int rc = check_common(fn, y, x, w_packed, scales_packed, n, k, group, dtype)) return rc;
  if (zeros_packed && (reinterpret_cast<uintptr_t>(zeros_packed) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: zeros must be 4-byte aligned", fn);
  if (m == 0) return KSQ_OK;
  if (m > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: m too large", fn);
  SplitKParams p{};
  p.y = y;
  p.x = x;
  p.w = static_cast<const u32x4*>(w_packed);
  p.scales = static_cast<const uint16_t*>(scales_packed);
  p.zeros = static_cast<const uint8_t*>(zeros_packed);
  p.M = static_cast<uint32_t>(m);
  p.N = static_cast<uint32_t>(n);
  p.K = static_cast<uint32_t>(k);
  SplitKChoice c = select_splitk(m, n, k);
  int rc = dtype == KSQ_F16 ? dispatch_tile<F16, false>(p, c, group, as_stream(stream))
                            : dispatch_tile<BF16, false>(p, c, group, as_stream(stream));
  if (rc) return rc;
  return check_launch(fn);
}

KSQ_EXPORT int ksq_moe_w4a16_gemm(void* out, const void* x, const void* w_packed, const void* scales_packed,
                                  const void* zeros_packed, const void* topk_w, const void* sorted_ids,
                                  const void* expert_ids, const void* num_post_pad, size_t numel, size_t top_k,
                                  size_t E, size_t n, size_t k, size_t group, size_t block_m, int dtype,
                                  void* stream) {
  const char* fn = "ksq_moe_w4a16_gemm";
  if (int rc = check_common(fn, out, x, w_packed, scales_packed, n, k, group, dtype)) return rc;
  if (!sorted_ids || !expert_ids || !num_post_pad) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null index buffer", fn);
  if (zeros_packed) return fail(KSQ_ERR_UNSUPPORTED, "%s: zero points are not supported for expert weights", fn);
  if (top_k == 0 || E == 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: top_k and E must be positive", fn);
  if (block_m != 16 && block_m != 32)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: block_m %zu not in {16,32}", fn, block_m);
  if (numel == 0) return KSQ_OK;
  const size_t cap_blocks = (numel + E * (block_m - 1)) / block_m;  // upper bound on aligned blocks
  if (cap_blocks > 65535) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: too many row blocks (%zu)", fn, cap_blocks);
  SplitKParams p{};
  p.y = out;
  p.x = x;
  p.w = static_cast<const u32x4*>(w_packed);
  p.scales = static_cast<const uint16_t*>(scales_packed);
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
  SplitKChoice c = select_splitk(block_m, n, k);
  c.mt = static_cast<int>(block_m / 16);
  int rc = dtype == KSQ_F16 ? dispatch_tile<F16, true>(p, c, group, as_stream(stream))
                            : dispatch_tile<BF16, true>(p, c, group, as_stream(stream));
  if (rc) return rc;
  return check_launch(fn);
}
