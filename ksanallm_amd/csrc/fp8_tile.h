// Prefill-regime blockwise-FP8 kernel (MFMA-bound): a workgroup of 8 wavefronts (2 along M x 4 along N) computes a
// 256 x 256 output tile over a contiguous range of 128-deep k-blocks.
//
//   - both operands are e4m3 bytes and need no conversion, so both go global -> LDS without touching registers
//     (global_load_lds_dwordx4), one 128-deep k-block (32 KiB of activations + 32 KiB of weights) per stage, two
//     stages.  A 16-row x 128-byte MFMA operand is a 2 KiB fragment read back with two ds_read_b128 per lane.
//     Activation fragments are filled from the row-major [m, k] bytes by two loads of 64 contiguous bytes per row,
//     their 16-byte pieces swizzled so that the read-back is free of bank conflicts; weight fragments arrive packed
//     (ksq_fp8_repack_weight) as two contiguous KiB and are read back in lane order.
//   - one v_mfma_f32_16x16x128_f8f6f4 covers exactly one scale block: its result goes to a scratch tile and is folded
//     into the accumulator with a_s[kb, m] * b_s[n/128, kb] by four fp32 FMAs, issued under the following MFMA.
//   - activation scales reach the lanes through LDS as well (one small LDS-targeted load per stage), the weight
//     scales of the workgroup's k range are staged there once: no per-lane scale loads in the loop.
//   - weights are the MFMA row operand, activations the column operand: a lane holds four consecutive output columns
//     of one token (8-byte stores) and needs one activation scale per row tile.
//   - the loads of the next k-block are issued from inline assembly under the first MFMAs of a stage; a single
//     `s_waitcnt vmcnt(0)` + barrier per stage makes them visible and releases the LDS slot that was just consumed.
#pragma once

#include "ksq_common.h"
#include "tile_work.h"

namespace ksq {

struct Fp8TileParams {
  const uint8_t* a;   // [m, k]
  const float* a_s;   // [k/128, m]
  const uint8_t* b;   // [n, k] in packed 2 KiB fragments (ksq_fp8_repack_weight)
  const float* b_s;   // [ceil(n/128), k/128]
  void* out;          // [m, n]
  float* out32;       // dense form, verification only: the fp32 sums go here, [m, n], and nothing is rounded to TO
  float* partial;     // [slot][part][256][256] fp32 tiles of the workgroups that compute a part of K
  uint32_t M, N, K;
  uint32_t tiles_m, tiles_n;
  uint32_t main_items, splits, kb_per_split;  // tile_work.h
  uint32_t as_row_bytes, as_kb_bytes;  // a_s[row, kb] at row * as_row_bytes + kb * as_kb_bytes: (4, 4*M) in the dense form
  // grouped (MoE) form: row block b = tile_m holds the slots sorted_ids[b*256 ..] of expert expert_ids[b]
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_w;
  uint32_t numel, top_k, scale_rows;  // scale_rows = ceil(N/128): rows of one expert's b_s
};

__device__ __forceinline__ f32x4 mfma_fp8_k128(i32x8 a, i32x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// GROUPED: the MoE form.  Row block tile_m is one 256-slot block of the aligned permutation: slot s reads activation
// row s / top_k (pad slots carry s >= numel) and that row's scales, weights and weight scales are those of expert
// expert_ids[tile_m], results go to out[s, :] (times topk_w[s] when given).  Blocks past num_post_pad leave at once;
// there is no cut along K in this form.
// WM = 8: 256-token tiles.  WM = 4: 128-token tiles (each wavefront 64 tokens x 64 weight rows) for row counts that
// would leave half of a 256-token tile to padding; a stage then holds 8 activation fragments.
constexpr int fp8_tile_stage_bytes(int wm) { return (2 * wm + 16) * 2048; }
// LDS stages: the 48 KiB stages of the 128-token tile fit three times, and need it - a stage of that tile is over in
// less time than a load takes to come back
constexpr int fp8_tile_stages(int wm) { return wm == 4 ? 3 : 2; }
constexpr size_t fp8_tile_lds_bytes(int wm, size_t kb_max) {
  return static_cast<size_t>(fp8_tile_stages(wm)) * (fp8_tile_stage_bytes(wm) + 1024) + 2 * kb_max * 4;
}

// BLOCK: slots between consecutive row blocks (tile_m * BLOCK is the block's first slot): the tile's own 32 * WM rows, or
// - grouped form - 256 for a 128-token tile that serves a 256-slot block of which at most the lower half holds tokens.
template <typename TO, bool GROUPED, int WM, int BLOCK>
__device__ __forceinline__ void fp8_tile_body(const Fp8TileParams& p, char* lds) {
  static_assert(WM == 8 || WM == 4, "256- or 128-token tiles");
  static_assert(BLOCK == 2 * WM * 16 || (GROUPED && WM == 4 && BLOCK == 256), "block stride");
  constexpr int WAVES_N = 4;
  constexpr int WN = 4;  // 16x16 tiles per wavefront: 16*WM tokens x 64 weight rows
  constexpr int BM = 2 * WM * 16, BN = 256;
  constexpr int FRAG = 2048;                  // bytes of one 16 x 128 operand fragment
  constexpr int AF = BM / 16;                 // activation fragments of a stage
  constexpr int AFW = AF / 4;                 // ... fetched by each of the wavefronts 0..3
  constexpr int STAGE_BYTES = fp8_tile_stage_bytes(WM);  // AF activation + 16 weight fragments
  constexpr int W_FRAG0 = AF;                 // first weight fragment of a stage
  constexpr int NS = fp8_tile_stages(WM);     // LDS stages

  const int lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15, lq = lane >> 4;
  const uint32_t KB = p.K / 128;

  // ---- work id (tile_work.h): output tile and the part of K this workgroup computes
  // (the divisions inside run on the vector unit: readfirstlane brings the wave-uniform results back to scalars)
  const TileWork work = tile_work(blockIdx.x, p.tiles_m, p.tiles_n, p.main_items, p.splits, GROUPED);
  const uint32_t tile_m = __builtin_amdgcn_readfirstlane(work.tile_m), tile_n = __builtin_amdgcn_readfirstlane(work.tile_n);
  const uint32_t part = __builtin_amdgcn_readfirstlane(work.part), slot = __builtin_amdgcn_readfirstlane(work.slot);
  const bool direct = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(work.direct)) != 0;
  const uint32_t m0 = tile_m * BLOCK, n0 = tile_n * BN;
  const uint32_t kb_begin = direct ? 0 : part * p.kb_per_split;
  const uint32_t kb_count = direct ? KB : ((KB - kb_begin) < p.kb_per_split ? (KB - kb_begin) : p.kb_per_split);

  // ---- operand staging.  Wavefronts 0..3 fetch the activation fragments 4w..4w+3, wavefronts 4..7 the weight
  // fragments 4(w-4)..+3.  An activation fragment (16 rows x 128 bytes) is two loads, one per 64-byte half h of the
  // rows; in a load four consecutive lanes take the four 16-byte pieces of one row (64 contiguous bytes: the granularity at which
  // the memory pipeline runs at full rate).  Load lane j lands at 1024h + 16j = 1024h + 64*(j/4) + 16*(j%4) and
  // fetches piece (j%4) ^ (j/16) of row j/4, so that MFMA lane (row r, k slot q) finds its two pieces 2(q%2)+p at
  // 1024*(q/2) + 64r + 16*((2(q%2)+p) ^ (r/4)): the sixteen lanes that read together hit different bank groups.
  size_t expert = 0;
  // Row tiles (16 tokens) of this block that hold tokens at all: the last block of the matrix may be short, and in the
  // grouped form an expert's last block is padded to the block size with the pad slots at its end.  A wavefront none
  // of whose row tiles holds a token (the upper half of a block that is at most half full) only takes its part in the
  // loads and barriers.
  uint32_t live_tiles = AF;
  if (!GROUPED) {
    const uint32_t rows = p.M - m0;
    live_tiles = rows < static_cast<uint32_t>(BM) ? (rows + 15) / 16 : AF;
  }
  if (GROUPED) {
    if (m0 >= static_cast<uint32_t>(p.num_post_pad[0])) return;  // uniform: the whole workgroup leaves
    expert = static_cast<size_t>(__builtin_amdgcn_readfirstlane(p.expert_ids[tile_m]));
    uint32_t rows = 0;
#pragma unroll
    for (int h = 0; h < BLOCK / 64; ++h) {
      const bool is_row = static_cast<uint32_t>(p.sorted_ids[m0 + h * 64 + lane]) < p.numel;
      rows += static_cast<uint32_t>(__builtin_popcountll(__builtin_amdgcn_ballot_w64(is_row)));
    }
    live_tiles = __builtin_amdgcn_readfirstlane((rows + 15) / 16);
  }
  // The two wavefront rows split the block's row tiles: WM each - or, when at most WM of the 2 * WM hold tokens (a
  // grouped block at most half full: an expert with half a block's slots), WM / 2 each of the lower WM, so that no SIMD
  // is left with one working wavefront and one that only takes part in loads and barriers.
  const bool lower_half = GROUPED && live_tiles <= WM;
  const uint32_t per_wave = lower_half ? WM / 2 : WM;  // row tiles a wavefront covers
  const uint32_t rt0 = wm * per_wave;                   // its first row tile
  const uint32_t mine = live_tiles > rt0 ? (live_tiles - rt0 < per_wave ? live_tiles - rt0 : per_wave) : 0;
  const bool idle = mine == 0;  // none of this wavefront's row tiles holds a token
  const bool stage_act = wave < 4;
  const uint32_t frag0 = (wave & 3) * (stage_act ? AFW : 4);
  // Weights come as packed 2 KiB fragments (ksq_fp8_repack_weight), fragment (strip, k-block) at (strip*KB + kb)*2048:
  // a half of a fragment is one contiguous KiB, fetched by one load with lane j taking bytes 16j, and lands in LDS as
  // it lies in memory - MFMA lane l then reads 16 bytes at 16l of each half, consecutive lanes consecutive addresses,
  // the one pattern the LDS serves at its full rate.
  const uint32_t k_step = stage_act ? 128u : 2048u;  // bytes from one k-block to the next
  const uint32_t strip0 = n0 / 16;
  const uint8_t* g_tile = stage_act ? p.a + static_cast<size_t>(GROUPED ? 0 : m0) * p.K
                                    : p.b + ((expert * (p.N / 16) + strip0) * KB) * 2048;
  g_tile += static_cast<size_t>(kb_begin) * k_step;
  const uint32_t row_limit = p.M - m0;  // token rows of this tile inside the matrix
  uint32_t d_voff[4], d_voff_hi[4];     // per fragment: first load, and second load minus its instruction offset of 64
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    if (stage_act && f >= AFW) {
      d_voff[f] = d_voff_hi[f] = 0;  // not fetched
    } else if (stage_act) {
      uint32_t row = (frag0 + f) * 16 + (lane >> 2);
      if (GROUPED) {
        uint32_t sid = static_cast<uint32_t>(p.sorted_ids[m0 + row]);
        sid = sid < p.numel ? sid : p.numel - 1;  // pad slots read some valid row; their results are dropped
        row = sid / p.top_k;
      } else {
        row = row < row_limit ? row : row_limit - 1;  // rows past the edge repeat the last row; their results are dropped
      }
      d_voff[f] = row * p.K + 16 * ((lane & 3) ^ (lane >> 4));
      d_voff_hi[f] = d_voff[f];
    } else {
      uint32_t strip = strip0 + frag0 + f;
      strip = strip < p.N / 16 ? strip : p.N / 16 - 1;  // strips past N repeat the last one; their results are dropped
      d_voff[f] = (strip - strip0) * KB * 2048 + 16 * lane;
      d_voff_hi[f] = d_voff[f] + 1024 - 64;
    }
  }
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char*)lds));
  const uint32_t d_lds = lds_base + ((stage_act ? 0 : W_FRAG0) + frag0) * FRAG;

  // ---- scales.  Activation scales of a k-block are 256 consecutive floats (a_s is token-contiguous): wavefronts 0..3
  // copy 64 of them each into LDS with one 4-byte-per-lane LDS-targeted load per stage.  The weight scales of the
  // workgroup's two 128-row scale blocks, for its whole k range, are copied into LDS once.  A lane needs one activation
  // scale per row tile (token = column l%16 of the MFMA result) and one weight scale per k-block.
  constexpr int SCALE_BASE = NS * STAGE_BYTES;    // [NS slots][256] activation scales, then [2][kb_count] weight scales
  constexpr int BS_BASE = SCALE_BASE + NS * 1024;
  // M % 4 == 0: wavefront 0 copies all 256 with one 16-byte-per-lane load (lanes whose four tokens lie past M repeat
  // the last four).  Otherwise wavefronts 0..3 copy 64 each, 4 bytes per lane, every lane clamped on its own.
  // (the one-load form needs the 256 scales of a k-block contiguous: dense form with token-contiguous scales)
  const bool s_vec = !GROUPED && (p.M & 3) == 0 && p.as_row_bytes == 4;
  uint32_t s_row = s_vec ? m0 + 4 * lane : m0 + (wave & 3) * 64 + lane;
  if (!s_vec && (wave & 3) * 64 >= BM) s_row = m0;  // this wavefront copies no scales (128-token tiles)
  if (GROUPED) {
    uint32_t sid = static_cast<uint32_t>(p.sorted_ids[s_row]);
    sid = sid < p.numel ? sid : p.numel - 1;
    s_row = sid / p.top_k;
  } else {
    const uint32_t s_last = s_vec ? p.M - 4 : p.M - 1;
    s_row = s_row < s_last ? s_row : s_last;
  }
  const uint32_t s_voff = s_row * p.as_row_bytes;
  const char* as_base = reinterpret_cast<const char*>(p.a_s) + static_cast<size_t>(kb_begin) * p.as_kb_bytes;
  const uint32_t s_lds = lds_base + SCALE_BASE + (s_vec ? 0 : (wave & 3) * 256);
  const uint32_t n_wave = n0 + wn * 64;
  {
    const uint32_t nb_last = (p.N - 1) / 128;
    for (uint32_t t = threadIdx.x; t < 2 * kb_count; t += 512) {
      const uint32_t blk = t / kb_count, kb = t - blk * kb_count;
      uint32_t nb = n0 / 128 + blk;
      nb = nb < nb_last ? nb : nb_last;
      reinterpret_cast<float*>(lds + BS_BASE)[t] = p.b_s[(expert * p.scale_rows + nb) * KB + kb_begin + kb];
    }
  }
  const float* bs_lds = reinterpret_cast<const float*>(lds + BS_BASE) + (wn >> 1) * kb_count;
  const float* as_lds = reinterpret_cast<const float*>(lds + SCALE_BASE) + rt0 * 16 + lrow;

  // Every group of loads is one assembly statement opening with `s_nop 4`: its scalar operands are in place before
  // it starts, and the wait states a vector memory instruction needs after a VALU write of a scalar register have
  // passed whatever produced them.
  auto load_scales = [&](uint32_t kb) {
    const uint32_t k = kb < kb_count ? kb : kb_count - 1;
    const char* ap = as_base + static_cast<size_t>(k) * p.as_kb_bytes;
    const uint32_t d = __builtin_amdgcn_readfirstlane(s_lds + (kb % NS) * 1024);
    if (s_vec) {
      if (wave == 0)
        asm volatile("s_nop 4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2" ::"v"(s_voff), "s"(d), "s"(ap)
                     : "memory", "m0");
    } else if (wave < BM / 64) {
      asm volatile("s_nop 4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, %2" ::"v"(s_voff), "s"(d), "s"(ap)
                   : "memory", "m0");
    }
  };
  // operands of k-block `kb` -> LDS slot kb % 2.  The instruction offset of an LDS-targeted load is added to the LDS
  // address as well as to the global one: the second half's 64-byte global offset is taken out of its LDS base.
  // (a block at most half full: the activation fragments of its upper half are never read and, where every wait is
  // for all of a wavefront's loads - two stages -, not fetched either)
  const bool skip_act = NS == 2 && lower_half && stage_act && frag0 >= static_cast<uint32_t>(WM);
  auto load_operands = [&](uint32_t kb) {
    if (skip_act) return;
    const uint32_t k = kb < kb_count ? kb : kb_count - 1;
    const uint8_t* src = g_tile + static_cast<size_t>(k) * k_step;
    const uint32_t f0 = __builtin_amdgcn_readfirstlane(d_lds + (kb % NS) * STAGE_BYTES);
    const uint32_t f0h = f0 + 1024 - 64;
    const uint32_t f1 = f0 + FRAG, f1h = f0h + FRAG;
    if (AFW == 2 && stage_act) {  // two activation fragments per wavefront (128-token tiles)
      asm volatile(
          "s_nop 4\n\t"
          "s_mov_b32 m0, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %8\n\t"
          "s_mov_b32 m0, %5\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %8 offset:64\n\t"
          "s_mov_b32 m0, %6\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %8\n\t"
          "s_mov_b32 m0, %7\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %8 offset:64"
          :
          : "v"(d_voff[0]), "v"(d_voff[1]), "v"(d_voff_hi[0]), "v"(d_voff_hi[1]), "s"(f0), "s"(f0h), "s"(f1), "s"(f1h),
            "s"(src)
          : "memory", "m0");
      return;
    }
    const uint32_t f2 = f1 + FRAG, f2h = f1h + FRAG;
    const uint32_t f3 = f2 + FRAG, f3h = f2h + FRAG;
    asm volatile(
        "s_nop 4\n\t"
        "s_mov_b32 m0, %8\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %16\n\t"
        "s_mov_b32 m0, %9\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %16 offset:64\n\t"
        "s_mov_b32 m0, %10\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %16\n\t"
        "s_mov_b32 m0, %11\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %5, %16 offset:64\n\t"
        "s_mov_b32 m0, %12\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %16\n\t"
        "s_mov_b32 m0, %13\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %6, %16 offset:64\n\t"
        "s_mov_b32 m0, %14\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %16\n\t"
        "s_mov_b32 m0, %15\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %7, %16 offset:64"
        :
        : "v"(d_voff[0]), "v"(d_voff[1]), "v"(d_voff[2]), "v"(d_voff[3]), "v"(d_voff_hi[0]), "v"(d_voff_hi[1]),
          "v"(d_voff_hi[2]), "v"(d_voff_hi[3]), "s"(f0), "s"(f0h), "s"(f1), "s"(f1h), "s"(f2), "s"(f2h), "s"(f3),
          "s"(f3h), "s"(src)
        : "memory", "m0");
  };
  // Everything this wavefront issued has landed, except the loads of the youngest stage when three stages are in use
  // (vmcnt retires in issue order; a wavefront issues the same loads every stage: 8 weight loads, or 2*AFW activation
  // loads with or without the one scale load in front of them).
  const bool has_scale_load = s_vec ? wave == 0 : wave < BM / 64;
  // This wavefront's fragment reads of the stage have returned: behind the barrier other wavefronts refill the slot they
  // came from, and a bare s_barrier waits for nothing by itself.
  auto reads_done = [&]() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };
  auto wait_stage = [&]() {
    if (NS == 2) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else if (!stage_act) {
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    } else if (has_scale_load) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * AFW + 1) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * AFW) : "memory");
    }
  };

  f32x4 acc[WN][WM];
#pragma unroll
  for (int t = 0; t < WN; ++t)
#pragma unroll
    for (int i = 0; i < WM; ++i) acc[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint32_t rd_lo = 1024 * (lq >> 1) + 64 * lrow + 16 * ((2 * (lq & 1)) ^ (lrow >> 2));
  const uint32_t rd_hi = rd_lo ^ 16;
  auto read_frag = [&](const char* base) {
    const i32x4 lo = *reinterpret_cast<const i32x4*>(base + rd_lo);
    const i32x4 hi = *reinterpret_cast<const i32x4*>(base + rd_hi);
    return i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  // weight fragments lie in LDS as packed: 16 bytes per lane in lane order, second half 1 KiB further
  auto read_wfrag = [&](const char* base) {
    const i32x4 lo = *reinterpret_cast<const i32x4*>(base + 16 * lane);
    const i32x4 hi = *reinterpret_cast<const i32x4*>(base + 1024 + 16 * lane);
    return i32x8{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  // one k-block: WMV * 4 MFMAs (WMV = this wavefront's row tiles that hold tokens); the scale FMAs of MFMA j are placed
  // after MFMA j+2 so that they run in its shadow, and the loads of k-block `next` (scales, then operands into the LDS
  // slot the previous stage used) are issued after the first MFMA.
  auto compute = [&](auto wmv_c, uint32_t slot, uint32_t kb, uint32_t next) {
    constexpr int WMV = decltype(wmv_c)::value;
    float sc[WMV];
    {
      const float bs = bs_lds[kb];
#pragma unroll
      for (int i = 0; i < WMV; ++i) sc[i] = as_lds[slot * 256 + i * 16] * bs;
    }
    const char* act = lds + slot * STAGE_BYTES + rt0 * FRAG;
    const char* wgt = lds + slot * STAGE_BYTES + (W_FRAG0 + wn * WN) * FRAG;
    i32x8 wf[WN];
    i32x8 af[2];
    wf[0] = read_wfrag(wgt);
    af[0] = read_frag(act);
#pragma unroll
    for (int t = 1; t < WN; ++t) wf[t] = read_wfrag(wgt + t * FRAG);
    __builtin_amdgcn_sched_barrier(0x4);
    f32x4 tmp[3];
    const f32x4 zero{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < WMV * WN + 2; ++j) {
      const int i = j / WN, t = j % WN;
      if (j < WMV * WN) {
        if (t == 0 && i + 1 < WMV) af[(i + 1) & 1] = read_frag(act + (i + 1) * FRAG);
        tmp[j % 3] = mfma_fp8_k128(wf[t], af[i & 1], zero);
      }
      __builtin_amdgcn_sched_barrier(0x4);
      if (j >= 2) {  // the MFMA issued two places earlier has left the pipeline by now
        const int pi = (j - 2) / WN, pt = (j - 2) % WN;
        const f32x4 r = tmp[(j - 2) % 3];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[pt][pi][e] = __builtin_fmaf(r[e], sc[pi], acc[pt][pi][e]);
      }
      __builtin_amdgcn_sched_barrier(0x4);  // keep MFMAs, FMAs and LDS reads in this order (scalar ALU may move)
      if (j == 0) {  // right behind the first MFMA: the longest flight time the two LDS stages allow
        load_scales(next);
        load_operands(next);
      }
    }
  };

  // ---- schedule: stage c computes k-block c out of LDS slot c % NS and, right behind its first MFMA, issues the loads
  // of k-block c+NS-1 into the slot stage c-1 used (every wavefront left it at the previous barrier).  At the end of
  // the stage the loads of k-block c+1 have to have landed; the barrier makes them visible to all wavefronts.
  load_scales(0);
  load_operands(0);
  if (NS == 3) {
    load_scales(1);
    load_operands(1);
  }
  wait_stage();
  __syncthreads();  // also publishes the weight-scale table written with ordinary stores above

  // The main loop exists once per number of this wavefront's row tiles that hold tokens: a padded row tile costs its
  // MFMAs' time on this SIMD and their power whether or not its results are stored.
  if (idle) {
    for (uint32_t c = 0; c < kb_count; ++c) {
      load_scales(c + NS - 1);
      load_operands(c + NS - 1);
      wait_stage();  // operands and scales of c+1
      reads_done();
      __builtin_amdgcn_s_barrier();
    }
  } else {
    for_tile_count<1, WM>(mine, [&](auto wmv_c) {
      for (uint32_t c = 0; c < kb_count; ++c) {
        compute(wmv_c, c % NS, c, c + NS - 1);
        wait_stage();  // operands and scales of c+1
        reads_done();
        __builtin_amdgcn_s_barrier();
      }
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // drain the clamped prefetches before the LDS is released

  // ---- store: lane holds token m = l%16 of the tile and weight rows (output columns) 4*(l/16) .. +3
  // Grouped form: the slot ids and routing weights of this lane's rows, fetched before the first store.  Read next to
  // each store they would wait for the stores in front of them (the compiler cannot know that the output does not
  // overlap the index arrays), one memory round trip after the other.
  uint32_t sids[WM];
  float rws[WM];
  if (GROUPED) {
#pragma unroll
    for (int i = 0; i < WM; ++i) sids[i] = static_cast<uint32_t>(p.sorted_ids[m0 + rt0 * 16 + (i < static_cast<int>(per_wave) ? i : 0) * 16 + lrow]);
#pragma unroll
    for (int i = 0; i < WM; ++i) rws[i] = (sids[i] < p.numel && p.topk_w) ? p.topk_w[sids[i]] : 1.0f;
  }
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    uint32_t row = m0 + rt0 * 16 + i * 16 + lrow;
    bool live = row < p.M && i < static_cast<int>(per_wave);  // row tiles past this wavefront's share belong to the other row
    float rw = 1.0f;
    if (GROUPED) {
      live = sids[i] < p.numel && i < static_cast<int>(per_wave);
      row = sids[i];
      rw = rws[i];
    }
    if (live) {
#pragma unroll
      for (int t = 0; t < WN; ++t) {
        const uint32_t ncol = n_wave + t * 16 + 4 * lq;
        if (ncol < p.N) {
          if (!GROUPED && direct && p.out32) {
            *reinterpret_cast<f32x4*>(p.out32 + static_cast<size_t>(row) * p.N + ncol) = acc[t][i];
          } else if (GROUPED || direct) {
            f32x4 v = acc[t][i];
            if (GROUPED) v *= rw;
            u32x2 o;
            o.x = pack2(TO::from_float(v[0]), TO::from_float(v[1]));
            o.y = pack2(TO::from_float(v[2]), TO::from_float(v[3]));
            *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(p.out) + static_cast<size_t>(row) * p.N + ncol) = o;
          } else {
            float* dst = p.partial + ((static_cast<size_t>(slot) * p.splits + part) * BM + (row - m0)) * BN + (ncol - n0);
            *reinterpret_cast<f32x4*>(dst) = acc[t][i];
          }
        }
      }
    }
  }
}

// A 256-slot block of the grouped form of which at most 128 slots hold tokens (an expert with half a block's tokens or
// fewer) runs the 128-token tile's code: three stages of 48 KiB instead of two of 64 - a half-empty stage is over in
// less time than its successor's loads take to arrive - and every wavefront at work.
template <typename TO, bool GROUPED = false, int WM = 8>
__global__ void __launch_bounds__(512, 1) fp8_tile_kernel(Fp8TileParams p) {
  extern __shared__ __attribute__((aligned(16))) char lds[];  // fp8_tile_lds_bytes (the larger of both forms)
  if constexpr (GROUPED && WM == 8) {
    const TileWork work = tile_work(blockIdx.x, p.tiles_m, p.tiles_n, p.main_items, p.splits, true);
    const uint32_t m0 = __builtin_amdgcn_readfirstlane(work.tile_m) * 256;
    if (m0 >= static_cast<uint32_t>(p.num_post_pad[0])) return;  // uniform: the whole workgroup leaves
    uint32_t rows = 0;
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const bool is_row = static_cast<uint32_t>(p.sorted_ids[m0 + h * 64 + (threadIdx.x & 63)]) < p.numel;
      rows += static_cast<uint32_t>(__builtin_popcountll(__builtin_amdgcn_ballot_w64(is_row)));
    }
    if (__builtin_amdgcn_readfirstlane(rows) <= 128) {
      fp8_tile_body<TO, true, 4, 256>(p, lds);
      return;
    }
  }
  fp8_tile_body<TO, GROUPED, WM, 2 * WM * 16>(p, lds);
}

}  // namespace ksq
