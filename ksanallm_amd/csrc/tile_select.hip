// Per-shape tile selection: closed-form rules of (kind, m, n, k, dtype) for a 256-CU, 8-XCD MI355X.
// Host code only; no timing and no device queries, so the answer is the same at load time and at run time.
#include "ksq_common.h"
#include "tile_select.h"

namespace ksq {

static constexpr int kNumCU = 256;

// Split-K wavefront kernel: every workgroup streams NT column tiles over the whole K.
// - WAVES: enough k-tiles per wavefront to keep a prefetch stage in flight, at most 16 wavefronts (1024 threads).
// - NT: two column tiles per workgroup halve the x-operand traffic out of L2, but only when that still leaves at
//   least two workgroups per CU.
SplitKChoice select_splitk(size_t m, size_t n, size_t k) {
  SplitKChoice c;
  c.mt = m <= 16 ? 1 : 2;
  const size_t kt = k / 128;
  c.waves = kt >= 32 ? 16 : 8;
  const size_t n_tiles = n / 16;
  c.nt = (n_tiles % 2 == 0 && n_tiles / 2 >= 2 * static_cast<size_t>(kNumCU)) ? 2 : 1;
  if (c.mt == 2 && c.nt == 2) c.waves = 8;  // 16 wavefronts leave 128 VGPRs each, too few for a 2x2 tile
  return c;
}

}  // namespace ksq

using namespace ksq;

KSQ_EXPORT int ksq_select_tile(int kind, size_t m, size_t n, size_t k, int dtype, ksq_tile_desc* d) {
  if (!d) return fail(KSQ_ERR_INVALID_ARGUMENT, "ksq_select_tile: null descriptor");
  if (m == 0 || n == 0 || k == 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "ksq_select_tile: empty problem");
  (void)dtype;
  *d = ksq_tile_desc{};
  switch (kind) {
    case KSQ_KIND_W4A16:
    case KSQ_KIND_MOE_W4A16: {
      SplitKChoice c = select_splitk(m, n, k);
      d->kernel = KSQ_KERNEL_SPLITK_WAVE;
      d->block_m = 16 * c.mt;
      d->block_n = 16 * c.nt;
      d->block_k = 128;
      d->waves = c.waves;
      d->split_k = c.waves;
      d->grid = static_cast<int32_t>((n / 16 / c.nt) * div_up(m, 16 * c.mt));
      return KSQ_OK;
    }
    case KSQ_KIND_FP8_BLOCKWISE:
      d->kernel = KSQ_KERNEL_MFMA_TILE;
      d->block_m = 16;
      d->block_n = 16;
      d->block_k = 128;
      d->waves = 4;
      d->split_k = 1;
      d->grid = static_cast<int32_t>(div_up(m, 16) * div_up(n, 16));
      return KSQ_OK;
    default:
      return fail(KSQ_ERR_INVALID_ARGUMENT, "ksq_select_tile: unknown kind %d", kind);
  }
}
