// Prefill-regime W4A8 kernel (MFMA-bound): a workgroup of 8 wavefronts (2 along M x 4 along N) computes a
// (32*WM) x 256 output tile over a contiguous range of 128-deep k-blocks (= scale groups) on the fp8 matrix instruction.
//
//   - activations (e4m3 bytes) and weights (packed int4 codes) both go global -> LDS without touching registers
//     (global_load_lds_dwordx4), one k-block per stage, three stages.  A 16-token x 128-byte activation operand is a
//     2 KiB fragment filled by two loads of 64 contiguous bytes per row, its 16-byte pieces swizzled so that the
//     read-back is free of bank conflicts; a weight fragment (16 columns x 128 k) is 1 KiB of codes, one contiguous
//     load, read back 16 bytes per lane in lane order and expanded to the 32 operand bytes with one shift and two ANDs
//     per dword (the byte 0x0u read as e4m3 is u * 2^-9).
//   - the per-token group sums ride the same kind of load into LDS; -xsum/64 is the instruction's addend, so its
//     result is 2^-9 * sum_k a_q * (u - 8) with no extra arithmetic.  The group's 256 fp16 weight scales are one more
//     LDS-targeted load per stage; a lane converts the four of its output columns per column tile and folds the
//     result into the accumulator with four fp32 FMAs, issued under the following MFMAs.
//   - weights are the MFMA row operand, activations the column operand: a lane holds four consecutive output columns
//     of one token (8-byte stores).
//   - the loads of a later k-block are issued from inline assembly under the first MFMA of a stage; one counted
//     `s_waitcnt vmcnt` + barrier per stage makes the next stage visible and releases the LDS slot just consumed.
#pragma once

#include "ksq_common.h"
#include "tile_work.h"

namespace ksq {

struct W4A8TileParams {
  const uint8_t* a;    // [m, k] e4m3
  const float* xsum;   // [k/128, m]
  const uint8_t* w;    // packed 1 KiB fragments (ksq_w4a8_repack_weight)
  const uint16_t* sc;  // fp16 [k/128, n]
  void* out;           // [m, n]
  float* partial;      // [slot][part][BM][256] fp32 tiles of the workgroups that compute a part of K
  uint32_t M, N, K;
  uint32_t tiles_m, tiles_n;
  uint32_t main_items, splits, kb_per_split;  // tile_work.h
  float alpha512;                             // alpha * 2^9
};

constexpr int w4a8_tile_stage_bytes(int wm) { return (2 * wm) * 2048 + 16 * 1024; }
constexpr int w4a8_tile_stages() { return 3; }
// per stage: operands, 1 KiB of group sums, 1 KiB of weight scales
constexpr size_t w4a8_tile_lds_bytes(int wm) {
  return static_cast<size_t>(w4a8_tile_stages()) * (w4a8_tile_stage_bytes(wm) + 2048);
}

__device__ __forceinline__ i32x8 w4a8_expand(i32x4 p) {
  i32x8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t w = static_cast<uint32_t>(p[i]);
    r[2 * i] = static_cast<int>(w & 0x0f0f0f0fu);
    r[2 * i + 1] = static_cast<int>((w >> 4) & 0x0f0f0f0fu);
  }
  return r;
}

// WM = 8: 256-token tiles.  WM = 4: 128-token tiles.
// GROUP = 64 (128-token tiles only): a k-block holds two scale groups.  Its two rows of group sums and of weight scales
// ride the same loads as the one row of GROUP = 128 (the lanes that repeat data there fetch the second row here), and
// every MFMA is issued twice, once with the weight bytes of the upper 64 k cleared and once with the lower ones
// cleared (this lane's 32 k lie in half lane / 32), each with its own addend and scales.
template <typename TO, int WM, int GROUP = 128>
__global__ void __launch_bounds__(512, 1) w4a8_tile_kernel(W4A8TileParams p) {
  static_assert(WM == 8 || WM == 4, "256- or 128-token tiles");
  static_assert(GROUP == 128 || (GROUP == 64 && WM == 4), "group 64 runs on 128-token tiles");
  constexpr int GH = 128 / GROUP;
  constexpr int WAVES_N = 4;
  constexpr int WN = 4;  // 16x16 tiles per wavefront: 16*WM tokens x 64 weight columns
  constexpr int BM = 2 * WM * 16, BN = 256;
  constexpr int FRAG = 2048;    // bytes of one 16-token x 128-byte activation fragment
  constexpr int WFRAG = 1024;   // bytes of one 16-column x 128-k weight fragment
  constexpr int AF = BM / 16;   // activation fragments of a stage
  constexpr int AFW = AF / 4;   // ... fetched by each of the wavefronts 0..3
  constexpr int STAGE_BYTES = w4a8_tile_stage_bytes(WM);
  constexpr int W_BASE = AF * FRAG;  // weight fragments of a stage start here
  constexpr int NS = w4a8_tile_stages();
  constexpr int XS_BASE = NS * STAGE_BYTES;    // [NS][256] group sums
  constexpr int WS_BASE = XS_BASE + NS * 1024;  // [NS][256 fp16 (+ 512 bytes unused)] weight scales

  extern __shared__ __attribute__((aligned(16))) char lds[];  // w4a8_tile_lds_bytes

  const int lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int lrow = lane & 15, lq = lane >> 4;
  const uint32_t KB = p.K / 128;

  const TileWork work = tile_work(blockIdx.x, p.tiles_m, p.tiles_n, p.main_items, p.splits);
  const uint32_t tile_m = __builtin_amdgcn_readfirstlane(work.tile_m), tile_n = __builtin_amdgcn_readfirstlane(work.tile_n);
  const uint32_t part = __builtin_amdgcn_readfirstlane(work.part), slot = __builtin_amdgcn_readfirstlane(work.slot);
  const bool direct = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(work.direct)) != 0;
  const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
  const uint32_t kb_begin = direct ? 0 : part * p.kb_per_split;
  const uint32_t kb_count = direct ? KB : ((KB - kb_begin) < p.kb_per_split ? (KB - kb_begin) : p.kb_per_split);

  // Row tiles (16 tokens) of this block that hold tokens at all (the last block of the matrix may be short).  A
  // wavefront none of whose row tiles holds a token only takes its part in the loads and barriers.
  const uint32_t rows_here = p.M - m0;
  const uint32_t live_tiles = rows_here < static_cast<uint32_t>(BM) ? (rows_here + 15) / 16 : AF;
  const bool idle = live_tiles <= wm * WM;

  // ---- operand staging.  Wavefronts 0..3 fetch the activation fragments AFW*w .. +AFW-1 (two loads each, one per
  // 64-byte half of the rows; load lane j lands at 1024h + 16j and fetches piece (j%4) ^ (j/16) of row j/4), wavefronts
  // 4..7 the weight fragments 4(w-4) .. +3 (one load each, lane j takes bytes 16j of the fragment).
  const bool stage_act = wave < 4;
  const uint32_t frag0 = (wave & 3) * (stage_act ? AFW : 4);
  const uint32_t k_step = stage_act ? 128u : 1024u;  // bytes from one k-block to the next
  const uint32_t strip0 = n0 / 16;
  const uint8_t* g_tile = stage_act ? p.a + static_cast<size_t>(m0) * p.K : p.w + (static_cast<size_t>(strip0) * KB) * 1024;
  g_tile += static_cast<size_t>(kb_begin) * k_step;
  uint32_t d_voff[4];
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    if (stage_act && f >= AFW) {
      d_voff[f] = 0;  // not fetched
    } else if (stage_act) {
      uint32_t row = (frag0 + f) * 16 + (lane >> 2);
      row = row < rows_here ? row : rows_here - 1;  // rows past the edge repeat the last row; their results are dropped
      d_voff[f] = row * p.K + 16 * ((lane & 3) ^ (lane >> 4));
    } else {
      uint32_t strip = strip0 + frag0 + f;
      strip = strip < p.N / 16 ? strip : p.N / 16 - 1;  // strips past N repeat the last one; their results are dropped
      d_voff[f] = (strip - strip0) * KB * 1024 + 16 * lane;
    }
  }
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char*)lds));
  const uint32_t d_lds = lds_base + (stage_act ? frag0 * FRAG : W_BASE + frag0 * WFRAG);

  // ---- group sums (tokens contiguous per k-block, like the activation scales of the blockwise kernel).  M % 4 == 0:
  // wavefront 0 copies the tile's BM values with one 16-byte-per-lane load (lanes whose four tokens lie past M repeat
  // the last four).  Otherwise wavefronts 0..BM/64-1 copy 64 each, 4 bytes per lane, every lane clamped on its own.
  const bool s_vec = (p.M & 3) == 0;
  uint32_t s_row = s_vec ? m0 + 4 * lane : m0 + (wave & 3) * 64 + lane;
  uint32_t s_half = 0;  // GROUP = 64: the lanes / wavefronts past the tile's tokens fetch the second row of sums
  if (s_vec && 4 * lane >= BM) {
    s_row = GH == 2 ? m0 + 4 * lane - BM : m0;
    s_half = GH == 2 ? 1 : 0;
  }
  if (!s_vec && (wave & 3) * 64 >= BM) {
    s_row = GH == 2 ? m0 + (wave & 3) * 64 + lane - BM : m0;
    s_half = GH == 2 ? 1 : 0;
  }
  {
    const uint32_t s_last = s_vec ? p.M - 4 : p.M - 1;
    s_row = s_row < s_last ? s_row : s_last;
  }
  const uint32_t s_voff = (s_half * p.M + s_row) * 4;
  const char* xs_base = reinterpret_cast<const char*>(p.xsum) + static_cast<size_t>(kb_begin) * GH * p.M * 4;
  const uint32_t s_lds = lds_base + XS_BASE + (s_vec ? 0 : (wave & 3) * 256);
  const bool has_xs_load = s_vec ? wave == 0 : wave < (GH == 2 ? 4 : BM / 64);
  // ---- weight scales of a k-block: 256 fp16 = 512 bytes, lanes 0..31 of wavefront 4 take 16 bytes (8 columns) each;
  // lanes 32..63 repeat them (their copy lands in the unused half of the slot)
  uint32_t ws_col = n0 + 8 * (lane & 31);
  ws_col = ws_col + 8 <= p.N ? ws_col : p.N - 8;
  const uint32_t ws_voff = (ws_col - n0) * 2 + ((GH == 2 && lane >= 32) ? p.N * 2 : 0);  // lanes 32..63: the second row
  const char* ws_base = reinterpret_cast<const char*>(p.sc) + (static_cast<size_t>(kb_begin) * GH * p.N + n0) * 2;
  const uint32_t ws_lds = lds_base + WS_BASE;
  const uint32_t n_wave = n0 + wn * 64;

  // Every group of loads is one assembly statement opening with `s_nop 4`: its scalar operands are in place before
  // it starts, and the wait states a vector memory instruction needs after a VALU write of a scalar register have
  // passed whatever produced them.
  auto load_scales = [&](uint32_t kb) {
    const uint32_t k = kb < kb_count ? kb : kb_count - 1;
    if (has_xs_load) {
      const char* ap = xs_base + static_cast<size_t>(k) * GH * p.M * 4;
      const uint32_t d = __builtin_amdgcn_readfirstlane(s_lds + (kb % NS) * 1024);
      if (s_vec)
        asm volatile("s_nop 4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2" ::"v"(s_voff), "s"(d), "s"(ap)
                     : "memory", "m0");
      else
        asm volatile("s_nop 4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, %2" ::"v"(s_voff), "s"(d), "s"(ap)
                     : "memory", "m0");
    }
    if (wave == 4) {
      const char* wp = ws_base + static_cast<size_t>(k) * GH * p.N * 2;
      const uint32_t d = __builtin_amdgcn_readfirstlane(ws_lds + (kb % NS) * 1024);
      asm volatile("s_nop 4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2" ::"v"(ws_voff), "s"(d), "s"(wp)
                   : "memory", "m0");
    }
  };
  // operands of k-block `kb` -> LDS slot kb % NS.  The instruction offset of an LDS-targeted load is added to the LDS
  // address as well as to the global one: the second half's 64-byte global offset is taken out of its LDS base.
  auto load_operands = [&](uint32_t kb) {
    const uint32_t k = kb < kb_count ? kb : kb_count - 1;
    const uint8_t* src = g_tile + static_cast<size_t>(k) * k_step;
    const uint32_t f0 = __builtin_amdgcn_readfirstlane(d_lds + (kb % NS) * STAGE_BYTES);
    if (!stage_act) {
      const uint32_t f1 = f0 + WFRAG, f2 = f1 + WFRAG, f3 = f2 + WFRAG;
      asm volatile(
          "s_nop 4\n\t"
          "s_mov_b32 m0, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %8\n\t"
          "s_mov_b32 m0, %5\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %8\n\t"
          "s_mov_b32 m0, %6\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %8\n\t"
          "s_mov_b32 m0, %7\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %8"
          :
          : "v"(d_voff[0]), "v"(d_voff[1]), "v"(d_voff[2]), "v"(d_voff[3]), "s"(f0), "s"(f1), "s"(f2), "s"(f3), "s"(src)
          : "memory", "m0");
      return;
    }
    const uint32_t f0h = f0 + 1024 - 64;
    const uint32_t f1 = f0 + FRAG, f1h = f0h + FRAG;
    if (AFW == 2) {  // two activation fragments per wavefront (128-token tiles)
      asm volatile(
          "s_nop 4\n\t"
          "s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %6\n\t"
          "s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %6 offset:64\n\t"
          "s_mov_b32 m0, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %6\n\t"
          "s_mov_b32 m0, %5\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %6 offset:64"
          :
          : "v"(d_voff[0]), "v"(d_voff[1]), "s"(f0), "s"(f0h), "s"(f1), "s"(f1h), "s"(src)
          : "memory", "m0");
      return;
    }
    const uint32_t f2 = f1 + FRAG, f2h = f1h + FRAG;
    const uint32_t f3 = f2 + FRAG, f3h = f2h + FRAG;
    asm volatile(
        "s_nop 4\n\t"
        "s_mov_b32 m0, %4\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %12\n\t"
        "s_mov_b32 m0, %5\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %12 offset:64\n\t"
        "s_mov_b32 m0, %6\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %12\n\t"
        "s_mov_b32 m0, %7\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %12 offset:64\n\t"
        "s_mov_b32 m0, %8\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %12\n\t"
        "s_mov_b32 m0, %9\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %12 offset:64\n\t"
        "s_mov_b32 m0, %10\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %12\n\t"
        "s_mov_b32 m0, %11\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %3, %12 offset:64"
        :
        : "v"(d_voff[0]), "v"(d_voff[1]), "v"(d_voff[2]), "v"(d_voff[3]), "s"(f0), "s"(f0h), "s"(f1), "s"(f1h), "s"(f2),
          "s"(f2h), "s"(f3), "s"(f3h), "s"(src)
        : "memory", "m0");
  };
  // Everything this wavefront issued has landed except the loads of the youngest stage (vmcnt retires in issue order;
  // a wavefront issues the same loads every stage: 4 weight loads with or without the weight-scale load, or 2*AFW
  // activation loads with or without the group-sum load).
  // This wavefront's fragment reads of the stage have returned: behind the barrier other wavefronts refill the slot they
  // came from, and a bare s_barrier waits for nothing by itself.
  auto reads_done = [&]() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };
  auto wait_stage = [&]() {
    if (!stage_act) {
      if (wave == 4)
        asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
      else
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    } else if (has_xs_load) {
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
  const float* xs_lds = reinterpret_cast<const float*>(lds + XS_BASE) + wm * (WM * 16) + lrow;
  const char* wsc_lds = lds + WS_BASE + (wn * 64 + 4 * lq) * 2;

  // one k-block: WM*WN MFMAs; the scale FMAs of MFMA j are placed after MFMA j+2 so that they run in its shadow, and
  // the loads of k-block `next` are issued after the first MFMA.
  auto compute = [&](uint32_t slot, uint32_t next) {
    if constexpr (GH == 2) {
      // group 64: sums of half h at [h][BM] floats, scales of half h at [h][256] fp16 of the stage's slots
      float cs[2][WM];
      float sc[2][WN][4];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int i = 0; i < WM; ++i) cs[h][i] = xs_lds[slot * 256 + h * BM + i * 16] * -0.015625f;
#pragma unroll
        for (int t = 0; t < WN; ++t) {
          const u32x2 v = *reinterpret_cast<const u32x2*>(wsc_lds + slot * 1024 + h * 512 + t * 32);
          sc[h][t][0] = F16::lo_to_float(v.x);
          sc[h][t][1] = F16::hi_to_float(v.x);
          sc[h][t][2] = F16::lo_to_float(v.y);
          sc[h][t][3] = F16::hi_to_float(v.y);
        }
      }
      const char* act = lds + slot * STAGE_BYTES + (wm * WM) * FRAG;
      const char* wgt = lds + slot * STAGE_BYTES + W_BASE + (wn * WN) * WFRAG + 16 * lane;
      i32x8 wf[2][WN];
      const int keep_lo = lane < 32 ? -1 : 0;
#pragma unroll
      for (int t = 0; t < WN; ++t) {
        const i32x8 w = w4a8_expand(*reinterpret_cast<const i32x4*>(wgt + t * WFRAG));
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          wf[0][t][e] = w[e] & keep_lo;
          wf[1][t][e] = w[e] & ~keep_lo;
        }
      }
#pragma unroll
      for (int i = 0; i < WM; ++i) {
        const i32x8 af = read_frag(act + i * FRAG);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const f32x4 cv{cs[h][i], cs[h][i], cs[h][i], cs[h][i]};
#pragma unroll
          for (int t = 0; t < WN; ++t) {
            const f32x4 r = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[h][t], af, cv, 0, 0, 0, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[t][i][e] = __builtin_fmaf(r[e], sc[h][t][e], acc[t][i][e]);
          }
        }
        if (i == 0) {
          load_scales(next);
          load_operands(next);
        }
      }
      return;
    }
    float cs[WM];
#pragma unroll
    for (int i = 0; i < WM; ++i) cs[i] = xs_lds[slot * 256 + i * 16] * -0.015625f;  // -8 * 2^-9 * xsum
    float sc[WN][4];
#pragma unroll
    for (int t = 0; t < WN; ++t) {
      const u32x2 h = *reinterpret_cast<const u32x2*>(wsc_lds + slot * 1024 + t * 32);
      sc[t][0] = F16::lo_to_float(h.x);
      sc[t][1] = F16::hi_to_float(h.x);
      sc[t][2] = F16::lo_to_float(h.y);
      sc[t][3] = F16::hi_to_float(h.y);
    }
    const char* act = lds + slot * STAGE_BYTES + (wm * WM) * FRAG;
    const char* wgt = lds + slot * STAGE_BYTES + W_BASE + (wn * WN) * WFRAG + 16 * lane;
    i32x8 wf[WN];
    i32x8 af[2];
    af[0] = read_frag(act);
#pragma unroll
    for (int t = 0; t < WN; ++t) wf[t] = w4a8_expand(*reinterpret_cast<const i32x4*>(wgt + t * WFRAG));
    __builtin_amdgcn_sched_barrier(0x4);
    f32x4 tmp[3];
    f32x4 cv[2];  // the addend of a row tile, spread once over the four registers the instruction reads
    cv[0] = f32x4{cs[0], cs[0], cs[0], cs[0]};
#pragma unroll
    for (int j = 0; j < WM * WN + 2; ++j) {
      const int i = j / WN, t = j % WN;
      if (j < WM * WN) {
        if (t == 0 && i + 1 < WM) {
          af[(i + 1) & 1] = read_frag(act + (i + 1) * FRAG);
          cv[(i + 1) & 1] = f32x4{cs[i + 1], cs[i + 1], cs[i + 1], cs[i + 1]};
        }
        tmp[j % 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[t], af[i & 1], cv[i & 1], 0, 0, 0, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0x4);
      if (j >= 2) {  // the MFMA issued two places earlier has left the pipeline by now
        const int pi = (j - 2) / WN, pt = (j - 2) % WN;
        const f32x4 r = tmp[(j - 2) % 3];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[pt][pi][e] = __builtin_fmaf(r[e], sc[pt][e], acc[pt][pi][e]);
      }
      __builtin_amdgcn_sched_barrier(0x4);  // keep MFMAs, FMAs and LDS reads in this order (scalar ALU may move)
      if (j == 0) {
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
  load_scales(1);
  load_operands(1);
  wait_stage();
  __syncthreads();

  for (uint32_t c = 0; c < kb_count; ++c) {
    if (idle) {
      load_scales(c + NS - 1);
      load_operands(c + NS - 1);
    } else {
      compute(c % NS, c + NS - 1);
    }
    wait_stage();  // operands and scales of c+1
    reads_done();
    __builtin_amdgcn_s_barrier();
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // drain the clamped prefetches before the LDS is released

  // ---- store: lane holds token m = l%16 of the tile and output columns 4*(l/16) .. +3
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const uint32_t row = m0 + wm * (WM * 16) + i * 16 + lrow;
    if (row < p.M) {
#pragma unroll
      for (int t = 0; t < WN; ++t) {
        const uint32_t ncol = n_wave + t * 16 + 4 * lq;
        if (ncol < p.N) {
          const f32x4 v = acc[t][i] * p.alpha512;
          if (direct) {
            u32x2 o;
            o.x = pack2(TO::from_float(v[0]), TO::from_float(v[1]));
            o.y = pack2(TO::from_float(v[2]), TO::from_float(v[3]));
            *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(p.out) + static_cast<size_t>(row) * p.N + ncol) = o;
          } else {
            float* dst = p.partial + ((static_cast<size_t>(slot) * p.splits + part) * BM + (row - m0)) * BN + (ncol - n0);
            *reinterpret_cast<f32x4*>(dst) = v;
          }
        }
      }
    }
  }
}

}  // namespace ksq
