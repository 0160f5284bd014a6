// Per-shape tile selection: closed-form rules of (kind, m, n, k, dtype) for a 256-CU, 8-XCD MI355X.
// Host code only; no timing and no device queries, so the answer is the same at load time and at run time.
#include <atomic>

#include "ksq_common.h"
#include "tile_select.h"

namespace ksq {

static constexpr int kNumCU = 256;

// ksq_set_small_problem_rule: 1 (default) lets small problems of more than 32 rows run the decode-form kernels
static std::atomic<int> g_small_problem_rule{1};

// Split-K wavefront kernel (decode regime, HBM-bound).  Measured on MI355X the kernel runs fastest with few, long
// lived wavefronts, each streaming a deep ring of loads, and with every workgroup resident from the first cycle:
// - 4 wavefronts per workgroup, wavefront w taking every 4th k-tile;
// - NT, the column tiles a wavefront streams per k-tile, as wide as the register file allows (8 for one 16-row tile
//   of x, 4 for two) while the grid still has about one workgroup per CU: the x fragments and the sum-of-x MFMA are
//   shared by the NT tiles, which also divides the x traffic out of L2 by NT.
// Dense form only: with a long K and few columns (k >= 2n: down / o projections) the grid-fill rule ends at narrow
// workgroups, every one of which fetches all of x - more bytes out of the L2 than the weights out of HBM once there are
// several rows.  Then 4 column tiles share the x fragments and K is cut over 2..8 workgroups to bring the workgroup
// count back to 160 or more (fp32 partial sums through the workspace, one small second pass).  The same helps when a
// wavefront's share of K is very long (k > 16384).  Measured on MI355X, e.g. n=4096 k=14336 m=32: 28 -> 16 us.
SplitKChoice select_splitk(size_t m, size_t n, size_t k) {
  const int mt = m <= 16 ? 1 : 2;
  const size_t m_blocks = div_up(m, 16 * mt);
  SplitKChoice c = select_splitk_blocks(mt, m_blocks, n, k);
  const size_t strips = n / 16;
  // several row blocks, and four column tiles per workgroup would put a second workgroup on some CUs only (those then
  // finish last): eight column tiles when that still leaves half the CUs a workgroup (n = k = 5120 at 128 rows)
  if (m_blocks >= 2 && c.nt == 4 && strips % 8 == 0 && strips / 4 * m_blocks > static_cast<size_t>(kNumCU) &&
      strips / 8 * m_blocks >= static_cast<size_t>(kNumCU) / 2)
    c.nt = 8;
  if (strips % 4 == 0 && c.nt < 4) {
    const size_t rows = m < static_cast<size_t>(16 * mt) ? m : static_cast<size_t>(16 * mt);
    const size_t x_bytes = rows * k * 2 * (strips / c.nt) * m_blocks;  // what all workgroups together read of x
    // K the long side: whenever x outweighs the weights.  Otherwise from 48 MB of x re-reads: below that the second
    // pass costs more than the traffic it saves (n = k = 5120: 16 tokens 13.8 -> 9.4 us, 32 tokens 22.1 -> 12.6 us;
    // n = k = 4096 at 8 tokens, 17 MB of re-reads, would go 5.5 -> 7.0 us)
    const bool long_k = k >= 2 * n && (x_bytes > k * n / 2 || k > 16384);
    const bool heavy_x = x_bytes >= (size_t(48) << 20);
    if (m_blocks >= 2 && !long_k && heavy_x) {
      // several row blocks: four column tiles with x through LDS (below) rather than a cut along K - the blocks already
      // fill the chip (n = k = 5120 at 64 rows: 19.2 -> 12 us; n = k = 4096: 10.7 -> 10.0 us)
      c.nt = 4;
    } else if (long_k || heavy_x) {
      int parts = 2;
      while (parts < 8 && strips / 4 * m_blocks * parts < 160) parts *= 2;
      while (parts > 1 && k / 128 / parts < 8) parts /= 2;
      if (parts > 1) {
        c.nt = 4;
        c.parts = parts;
      }
    }
  }
  // x through LDS (group 128 only; the caller falls back to the register form otherwise).  Measured on MI355X:
  // - 17..32 rows: the x fragments are twice the weights' bytes, and fetched as 64-byte pieces of 32 rows they cost
  //   more than the weights (n = 25600, k = 5120: 27.4 -> 21.7 us; n = 14336, k = 4096: 12.8 -> 11.5 us);
  // - up to 16 rows: pays from about 48 MB of weights (n = 57344, k = 8192: 1 row 41.9 -> 40.7 us, 16 rows
  //   47.8 -> 46.3 us; n = 25600, k = 5120 at 16 rows 15.9 -> 15.0 us), not below (n = 14336, k = 4096 at 8 rows:
  //   7.9 us in registers, 8.4 us through LDS), and with up to 8 rows four column tiles per wavefront beat eight
  //   (n = 57344, k = 8192, 1 row: 40.7 against 43.1 us).
  if (c.parts == 1 && strips % 4 == 0) {
    if (mt == 2 && c.nt == 8) {
      c.waves = 4;
      c.xc = 4;
    } else if (mt == 2 && c.nt == 4) {
      c.waves = 8;
      c.xc = 8;
    } else if (mt == 1 && c.nt >= 4 && n * k / 2 >= (size_t(48) << 20)) {
      if (m <= 8) c.nt = 4;
      c.waves = 8;
      c.xc = 8;
    }
  }
  return c;
}

SplitKChoice select_splitk_blocks(int mt, size_t m_blocks, size_t n, size_t k) {
  SplitKChoice c;
  c.mt = mt;
  c.waves = 4;
  c.nt = 1;
  c.parts = 1;
  c.xc = 0;
  const size_t n_tiles = n / 16;
  // (eight column tiles also with two row tiles: n = 25600, k = 5120 at 32 rows 29.0 -> 22.4 us - half the x re-reads)
  for (int nt = 8; nt > 1; nt >>= 1) {
    if (n_tiles % nt == 0 && n_tiles / nt * m_blocks >= static_cast<size_t>(kNumCU) * 3 / 4) {
      c.nt = nt;
      break;
    }
  }
  (void)k;
  return c;
}

// Regime switch.  Up to 32 rows the split-K (decode) kernel; above, the MFMA tile kernel - except while the problem is
// small: the tile kernel has a floor of 17-22 us (a workgroup's prologue, the fp32 partial tiles of the cut along K and
// the pass that sums them), and the decode kernel run over blocks of 32 rows, each streaming the weights again (out of
// the L2: the blocks of one column group run on one XCD at the same time), stays below it while
// ceil(m / 32) * n * k <= 2^28, or 2^27 when K is the long side by four times or more (every block then re-reads a long
// row of x per column group).  Measured on MI355X over twelve shapes and 48..512 rows, decode / tile kernel in us:
// n = k = 4096 at 64 rows 10.9 / 19.2, at 128 rows 10.8 / 25.6, at 512 rows 27.0 / 29.5; n = 8192, k = 2048 at 128 rows
// 11.3 / 26.4, at 512 rows 29.2 / 40.1; n = k = 8192 at 64 rows 18.1 / 24.1, at 128 rows 30.6 / 32.0, at 192 rows
// 44.4 / 41.3; n = 14336, k = 4096 at 64 rows 17.9 / 23.1, at 128 rows 26.4 / 30.3, at 384 rows 75.1 / 56.3; n = 4096,
// k = 14336 at 128 rows 27.9 / 32.1, at 192 rows 48.4 / 38.9; n = 25600, k = 5120 at 64 rows 33.5 / 37.6, at 96 rows
// 48.6 / 46.1; n = 4096, k = 28672 at 64 rows 35.8 / 34.4; n = 5120, k = 25600 at 64 rows 61.7 / 36.6.
// (Group 128 only: the wide decode instances exist for that group.)
bool small_w4a16_problem(size_t m, size_t n, size_t k, size_t group) {
  const size_t limit = k >= 4 * n ? (size_t(1) << 27) : (size_t(1) << 28);
  return group == 128 && m <= kRowBlockMaxM && div_up(m, 32) * n * k <= limit;
}
bool use_mfma_tile(size_t m, size_t n, size_t k, size_t group) {
  if (m <= 32 || !(group == 128 || group == 64 || group == 32)) return false;
  if (g_small_problem_rule.load(std::memory_order_relaxed) && small_w4a16_problem(m, n, k, group)) return false;
  return true;
}

// 256-row tiles halve the weight traffic per output row, 128-row tiles waste less when m sits just above a multiple
// of 256.  With fewer than 192 output tiles the k range is cut into up to 256/tiles pieces of at least 4 k-tiles (512 k)
// each; the fp32 partial tiles are summed by a second, bandwidth-bound kernel.
// How to spread `tiles` output tiles of `kt` k-steps over the CUs.  Costs are in k-steps of one workgroup:
//   fixed    prologue + epilogue of a workgroup
//   partial  storing an fp32 partial tile instead of the output tile (and reading it back in the reduction)
//   reduce   launch of the reduction pass, plus per_unit for every partial tile it reads
// Candidates: every tile whole (ceil(tiles/CUs) rounds), or the full rounds whole and the tiles of the last, partly
// filled round cut into s parts of K.  A part is at least 4 k-steps and at most 512 partial tiles are written.
struct SpreadCost {
  double fixed, partial, reduce, per_unit;
};

void spread_tiles(unsigned tiles, unsigned kt, const SpreadCost& c, TilePlan* t) {
  const unsigned cus = static_cast<unsigned>(kNumCU);
  const unsigned full = tiles / cus * cus, rem = tiles - full;
  double best = div_up(tiles, cus) * (kt + c.fixed);
  t->main_items = 0;
  t->splits = 1;
  t->kt_per_split = kt;
  if (rem == 0) return;
  for (unsigned s = 2; s <= 16; ++s) {
    const unsigned per = static_cast<unsigned>(div_up(kt, s));
    if (per < 4) break;
    if (div_up(kt, per) != s) continue;  // the same parts as a smaller s
    const unsigned units = rem * s;
    if (units > 512) break;
    const double cost = (full / cus) * (kt + c.fixed) + div_up(units, cus) * (per + c.fixed + c.partial) + c.reduce + units * c.per_unit;
    if (cost < best) {
      best = cost;
      t->main_items = full;
      t->splits = s;
      t->kt_per_split = per;
    }
  }
}

void finish_plan(TilePlan* t) {
  const unsigned tiles = t->tiles_m * t->tiles_n;
  const unsigned cut = t->splits > 1 ? tiles - t->main_items : 0;
  t->grid = t->main_items + (tiles - t->main_items) * t->splits;
  t->workspace_bytes = static_cast<size_t>(cut) * t->splits * t->block_m * 256 * sizeof(float);
}

TilePlan plan_mfma_tile(size_t m, size_t n, size_t k) {
  TilePlan t{};
  const size_t rem = (m - 1) % 256;
  t.block_m = (m <= 128 || (m < 1024 && rem < 128)) ? 128 : 256;
  t.tiles_n = static_cast<unsigned>(div_up(n, 256));
  // where 256-row tiles leave more than half of the CUs idle but 128-row tiles fill the grid, take those (the weights are then fetched
  // twice as often, out of the L2 / Infinity Cache) rather than split K: fp32 partial tiles cost 8 bytes of HBM
  // traffic per output element and split.  Where neither fills it, 256-row tiles with a deeper split measured faster.
  const unsigned fill = static_cast<unsigned>(kNumCU) * 3 / 4;
  if (t.block_m == 256 && div_up(m, 256) * t.tiles_n < static_cast<unsigned>(kNumCU) / 2 && div_up(m, 128) * t.tiles_n >= fill)
    t.block_m = 128;
  // very few 256-row tiles (at most 32) are cut so finely along K that their fp32 partial tiles outweigh what the
  // larger tile saves: 128-row tiles need half the cut (n = k = 4096: 256 rows 34 -> 27 us, 512 rows 42 -> 33 us;
  // n = 4096, k = 14336 at 256 rows 52 -> 45 us; with K beyond 16384 the larger tile stays 1-3 % ahead)
  if (t.block_m == 256 && div_up(m, 256) * t.tiles_n <= 32 && k <= 16384) t.block_m = 128;
  t.tiles_m = static_cast<unsigned>(div_up(m, t.block_m));
  static const SpreadCost cost{3.0, 3.0, 2.0, 0.02};
  spread_tiles(t.tiles_m * t.tiles_n, static_cast<unsigned>(k / 128), cost, &t);
  finish_plan(&t);
  return t;
}

// Above two 16-token tiles the MFMA tile kernel (with split-K) - except, as for W4A16, while the problem is small enough
// for the streaming kernel over blocks of 32 tokens (four strips per workgroup sharing a block's activation fragments)
// to stay below the tile kernel's floor (15-22 us): ceil(m / 32) * n * k <= 5 * 2^24, and not with a K so short that a
// workgroup's life is its prologue (n > 4 k).  Measured on MI355X over eleven shapes and 48..512 tokens, streaming / tile
// kernel in us: n = k = 4096 at 64 tokens 11.3 / 17.5, at 128 tokens 11.2 / 22.4, at 256 tokens 20.1 / 23.0, at 384
// tokens 28.5 / 23.8; n = 2048, k = 7168 at 128 tokens 16.0 / 23.1, at 256 tokens 16.0 / 22.2, at 384 tokens 29.2 / 23.4;
// n = 7168, k = 2048 at 192 tokens 18.9 / 23.6, at 256 tokens 24.0 / 23.6; n = 4608, k = 7168 at 64 tokens 17.1 / 18.7, at
// 128 tokens 31.9 / 22.3; n = 7168, k = 4608 at 64 tokens 13.6 / 18.0, at 96 tokens 25.0 / 20.0; n = k = 7168 at 64 tokens
// 18.2 / 21.0, at 96 tokens 33.6 / 22.9; n = 24576, k = 1536 at 64 tokens 22.0 / 19.6; n = 18432, k = 7168 at 48 tokens
// 52.9 / 32.1.
bool use_fp8_tile(size_t m, size_t n, size_t k) {
  if (m <= 32) return false;
  if (g_small_problem_rule.load(std::memory_order_relaxed) && m <= kRowBlockMaxM && n <= 4 * k &&
      div_up(m, 32) * n * k <= (size_t(5) << 24))
    return false;
  return true;
}

// W4A8: the same, with the limit where its two kernels cross: ceil(m / 32) * n * k <= 5 * 2^25 (n <= 4 k).  Measured on
// MI355X over nine shapes and 48..512 tokens, streaming / tile kernel in us: n = k = 4096 at 64 tokens 9.5 / 16.9, at 128
// tokens 10.5 / 24.1, at 256 tokens 15.3 / 24.1, at 512 tokens 35.0 / 26.0; n = k = 5120 at 96 tokens 11.7 / 22.8, at 192
// tokens 18.7 / 23.6, at 256 tokens 28.5 / 24.6; n = 8192, k = 2048 at 128 tokens 10.3 / 23.6; n = 2048, k = 7168 at 256
// tokens 16.4 / 22.0; n = k = 8192 at 64 tokens 18.1 / 20.0, at 96 tokens 26.1 / 24.7; n = 14336, k = 4096 at 64 tokens
// 15.6 / 18.7, at 96 tokens 23.7 / 23.7; n = 25600, k = 5120 at 48 tokens 32.8 / 27.1.
bool use_w4a8_tile(size_t m, size_t n, size_t k) {
  if (m <= 32) return false;
  if (g_small_problem_rule.load(std::memory_order_relaxed) && m <= kRowBlockMaxM && n <= 4 * k &&
      div_up(m, 32) * n * k <= (size_t(5) << 25))
    return false;
  return true;
}

TilePlan plan_fp8_tile(size_t m, size_t n, size_t k) {
  TilePlan t{};
  // 128-token tiles where 256-token ones would be half padding (the weights are then fetched once per 128 tokens);
  // with full tiles the 256-token form is faster (M = 4096: 509 against 641 us)
  t.block_m = (m <= 128 || (m < 1024 && (m - 1) % 256 < 128)) ? 128 : 256;
  // as in plan_mfma_tile: at most 32 tiles of 256 tokens are better served by 128-token tiles and half the cut along K
  // (n = k = 5120 at 256 tokens: 31 -> 25 us; n = k = 4096 at 512 tokens: 33 -> 27 us)
  if (t.block_m == 256 && div_up(m, 256) * div_up(n, 256) <= 32 && k <= 16384) t.block_m = 128;
  t.tiles_m = static_cast<unsigned>(div_up(m, t.block_m));
  t.tiles_n = static_cast<unsigned>(div_up(n, 256));
  // fitted over five shapes at 64..2048 tokens; costlier cuts had left n = 25600, k = 5120 at 64..256 tokens on 100
  // of the 256 CUs (48 / 50 / 78 us against 36 / 43 / 65 us cut in two)
  static const SpreadCost cost{6.0, 4.0, 3.0, 0.035};
  spread_tiles(t.tiles_m * t.tiles_n, static_cast<unsigned>(k / 128), cost, &t);
  finish_plan(&t);
  return t;
}

// W4A8: the blockwise-FP8 tile shapes; a k-step moves three quarters of the bytes and its prologue is shorter, so a
// cut along K pays earlier (measured at n = 25600, k = 5120: with the FP8 costs 64 / 128 / 256 tokens ran whole tiles
// on 100 of the 256 CUs in 38 / 51 / 83 us, with these they are cut in two or three: 28 / 38 / 60 us)
TilePlan plan_w4a8_tile(size_t m, size_t n, size_t k) {
  TilePlan t{};
  t.block_m = (m <= 128 || (m < 1024 && (m - 1) % 256 < 128)) ? 128 : 256;
  // as in plan_mfma_tile: at most 32 tiles of 256 tokens are better served by 128-token tiles and half the cut along K
  // (n = k = 5120 at 256 tokens: 31 -> 25 us; n = k = 4096 at 512 tokens: 33 -> 27 us)
  if (t.block_m == 256 && div_up(m, 256) * div_up(n, 256) <= 32 && k <= 16384) t.block_m = 128;
  t.tiles_m = static_cast<unsigned>(div_up(m, t.block_m));
  t.tiles_n = static_cast<unsigned>(div_up(n, 256));
  static const SpreadCost cost{6.0, 4.0, 3.0, 0.03};
  spread_tiles(t.tiles_m * t.tiles_n, static_cast<unsigned>(k / 128), cost, &t);
  finish_plan(&t);
  return t;
}

// W4A8 decode: a workgroup takes as many 16-column strips (up to 4) as still leave 128 workgroups - counting the row
// blocks of a problem of more than 32 tokens: n = k = 5120 at 64 tokens 16.8 -> 11.4 us with four strips instead of
// two -, and splits K over 8 wavefronts instead of 4 when fewer than 256 workgroups are left.
SplitKChoice select_w4a8_splitk(size_t m, size_t n) {
  SplitKChoice c{};
  c.mt = m <= 16 ? 1 : 2;
  c.nt = 4;
  const size_t m_blocks = div_up(m, 16 * c.mt);
  while (c.nt > 1 && (n % (16 * c.nt) != 0 || n / (16 * c.nt) * m_blocks < 128)) c.nt /= 2;
  c.waves = n / (16 * c.nt) * m_blocks < 256 ? 8 : 4;
  c.parts = 1;
  c.xc = 0;
  return c;
}

}  // namespace ksq

using namespace ksq;

// The same for block-fp8 experts (ksq_moe_fp8_blockwise_gemm): 16- and 32-row blocks stream through the split-K
// kernel; from 16 rows per expert the MFMA tile kernel is faster even with most of a 128-row block padding (each of its
// wavefronts multiplies the row tiles that hold rows), and 256-row blocks take over from 128 rows per expert, where an
// expert would otherwise need a second block and its weights a second pass.  E = 256, hidden 7168, inter 2048, top-8,
// whole call with 16- / 32- / 128- / 256-row blocks: 1.50 / 1.49 / 1.61 / - ms at 2 rows per expert, 1.85 / 1.84 /
// 1.95 / - at 8, 2.08 / 1.94 / 1.97 / - at 12, 2.60 / 2.06 / 2.01 / 2.46 at 16, - / 3.21 / 2.16 / 2.46 at 32,
// - / 5.51 / 2.37 / 2.66 at 64, - / 9.89 / 3.36 / 3.33 at 128, - / - / 4.23 / 3.84 at 192, - / - / 5.46 / 5.07 at 256.
KSQ_EXPORT size_t ksq_moe_fp8_block_m(size_t numel, size_t E) {
  if (E == 0) return 16;
  const size_t per_expert = numel / E;
  if (per_expert >= 128) return 256;
  if (per_expert >= 16) return 128;
  return per_expert < 2 ? 16 : 32;
}

// Rows per expert block for numel routed (token, slot) pairs over E experts.  Replaces the M thresholds of
// InvokeFusedMoe (16 / 32 / 64 rows by token count): below about 40 rows per expert the weights are streamed once per
// 16- or 32-row block (HBM-bound); above, the MFMA tile kernel takes 256-row blocks, of which it multiplies the row
// tiles that hold rows (an instance of its main loop per count), so that an expert's weights are dequantized once
// however many of the 256 rows it fills.  E = 256, hidden 7168, inter 2048, top-8, whole call with 32- / 128- /
// 256-row blocks: 1.97 / 2.34 / 2.37 ms at 32 rows per expert, 2.41 / 2.40 / 2.39 at 40, 2.58 / 2.46 / 2.45 at 48,
// 3.21 / 2.60 / 2.55 at 64, 4.39 / 3.06 / 3.02 at 96, 4.96 / 3.44 / 3.30 at 112, 5.60 / 4.40 / 3.57 at 128.
KSQ_EXPORT size_t ksq_moe_block_m(size_t numel, size_t E) {
  if (E == 0) return 16;
  const size_t per_expert = numel / E;
  if (per_expert >= 40) return 256;
  return per_expert < 16 ? 16 : 32;
}

KSQ_EXPORT int ksq_set_small_problem_rule(int enabled) { return g_small_problem_rule.exchange(enabled ? 1 : 0); }

KSQ_EXPORT int ksq_select_tile(int kind, size_t m, size_t n, size_t k, int dtype, ksq_tile_desc* d) {
  if (!d) return fail(KSQ_ERR_INVALID_ARGUMENT, "ksq_select_tile: null descriptor");
  if (m == 0 || n == 0 || k == 0) return fail(KSQ_ERR_INVALID_ARGUMENT, "ksq_select_tile: empty problem");
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "ksq_select_tile: dtype %d has no kernel", dtype);
  if (k % 128 != 0 || n % 16 != 0)
    return fail(KSQ_ERR_UNSUPPORTED, "ksq_select_tile: no kernel for n=%zu k=%zu (k must be a multiple of 128, n of 16)", n, k);
  *d = ksq_tile_desc{};
  switch (kind) {
    case KSQ_KIND_W4A16:
    case KSQ_KIND_MOE_W4A16: {
      if (kind == KSQ_KIND_W4A16 && use_mfma_tile(m, n, k, 128)) {
        const TilePlan t = plan_mfma_tile(m, n, k);
        d->kernel = KSQ_KERNEL_MFMA_TILE;
        d->block_m = t.block_m;
        d->block_n = 256;
        d->block_k = 64;
        d->waves = 8;
        d->split_k = static_cast<int32_t>(t.splits);
        d->grid = static_cast<int32_t>(t.grid);
        return KSQ_OK;
      }
      SplitKChoice c = select_splitk(m, n, k);
      d->kernel = KSQ_KERNEL_SPLITK_WAVE;
      d->block_m = 16 * c.mt;
      d->block_n = 16 * c.nt;
      d->block_k = 128;
      d->waves = c.waves;
      d->split_k = c.waves * c.parts;
      d->grid = static_cast<int32_t>((n / 16 / c.nt) * div_up(m, 16 * c.mt) * c.parts);
      d->x_chunk = kind == KSQ_KIND_W4A16 ? c.xc : 0;
      return KSQ_OK;
    }
    case KSQ_KIND_FP8_BLOCKWISE: {
      if (use_fp8_tile(m, n, k)) {
        const TilePlan t = plan_fp8_tile(m, n, k);
        d->kernel = KSQ_KERNEL_MFMA_TILE;
        d->block_m = t.block_m;
        d->block_n = 256;
        d->block_k = 128;
        d->waves = 8;
        d->split_k = static_cast<int32_t>(t.splits);
        d->grid = static_cast<int32_t>(t.grid);
        return KSQ_OK;
      }
      // decode: 16 weight rows x (16|32|64) tokens per workgroup, the wavefronts split K between them
      const int mt = m <= 16 ? 1 : 2;
      const int waves = 4;
      d->kernel = KSQ_KERNEL_SPLITK_WAVE;
      int nt = ((m > 8 || k > n) && n % 32 == 0) ? 2 : 1;
      if (m > 32 && n % 64 == 0 && n / 64 * div_up(m, 32) >= 128) nt = 4;  // as fp8_blockwise_gemm.hip's dispatch
      d->block_m = 16 * mt;
      d->block_n = 16 * nt;
      d->block_k = 128;
      d->waves = waves;
      d->split_k = waves;
      d->grid = static_cast<int32_t>(div_up(m, 16 * mt) * (n / (16 * nt)));
      return KSQ_OK;
    }
    case KSQ_KIND_W4A8: {
      if (use_w4a8_tile(m, n, k)) {
        const TilePlan t = plan_w4a8_tile(m, n, k);
        d->kernel = KSQ_KERNEL_MFMA_TILE;
        d->block_m = t.block_m;
        d->block_n = 256;
        d->block_k = 128;
        d->waves = 8;
        d->split_k = static_cast<int32_t>(t.splits);
        d->grid = static_cast<int32_t>(t.grid);
        return KSQ_OK;
      }
      const SplitKChoice c = select_w4a8_splitk(m, n);
      d->kernel = KSQ_KERNEL_SPLITK_WAVE;
      d->block_m = 16 * c.mt;
      d->block_n = 16 * c.nt;
      d->block_k = 128;
      d->waves = c.waves;
      d->split_k = c.waves;
      d->grid = static_cast<int32_t>(div_up(m, 16 * c.mt) * (n / (16 * c.nt)));
      return KSQ_OK;
    }
    default:
      return fail(KSQ_ERR_INVALID_ARGUMENT, "ksq_select_tile: unknown kind %d", kind);
  }
}
