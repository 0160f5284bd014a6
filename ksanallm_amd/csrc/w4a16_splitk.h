// Decode-regime W4A16 kernel (small M, HBM-bound).
//
// Work decomposition
//   grid.x : groups of NT column tiles (16 output columns each)
//   grid.y : blocks of MT*16 rows of x (MoE: aligned blocks of sorted slots, one expert each)
//   grid.z : parts of K (dense form, shapes with few columns and a long K: wide workgroups share the x fragments over
//            NT column tiles, and the parts of K bring the number of workgroups back up)
// Wavefront w of a workgroup takes the 128-wide k-tiles w, w+WAVES, ...
// Per k-tile a wavefront loads the x operand once (MT*4 fragments of 16 bytes per lane) and streams the NT weight
// tiles of that k-tile, one coalesced 1 KiB wavefront load each.  Every packed dword becomes an MFMA operand holding
// magic+code with seven bit operations, x is the row operand and the weights the column operand of
// v_mfma_f32_16x16x32, so a lane's four results share one output column, hence one scale and one zero point:
//     acc += s * (sum_k x*(magic+code) - (magic+zp) * sum_k x)
// with sum_k x from one more MFMA against an all-ones operand, shared by the NT tiles.  Without zero points that MFMA
// multiplies by -(magic + 8) itself and the weight MFMAs accumulate on top of its result: acc += s * r.
//
// What bounds the kernel is HBM latency x bandwidth, so the loads of a wavefront form one ring in issue order
// (vmcnt retires loads in order: a second, shallower ring would drain the first each time it is waited for).  The
// ring holds LOOK k-tiles ahead, NT weight tiles plus the x fragments each, sized so that a CU keeps 64 KiB or more
// in flight; buffer loads with a scalar offset keep address arithmetic off the VALU.
//
// The wavefronts' partials meet in LDS and are summed in wavefront order: the summation order is fixed, so the
// output does not depend on timing.
//
// Rows of x beyond M are not fetched at all (buffer loads past the extent of the resource return zero): an MFMA output
// row depends only on its own row of x, and those rows are never stored.
#pragma once

#include <type_traits>

#include "ksq_common.h"
#include "splitk_reduce.h"

namespace ksq {

struct SplitKParams {
  void* y;
  const void* x;
  const void* w;
  const void* scales;
  const void* zeros;
  uint32_t M, N, K;
  // grouped (MoE) mode
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_w;
  uint32_t numel, top_k;
  // K cut over grid.z workgroups as well (dense form): part z covers k-tiles [z*kt_per_part, ...) and writes fp32
  // partial sums [z][M][N] instead of the output; a second pass (parts_reduce_kernel) adds them up in the order of z.
  // (Summing them in the workgroup that finishes last, found with an arrival counter, measured slower than the second
  // launch: partial results that cross XCDs have to go through memory with device-scope stores, an atomic and
  // device-scope loads, three dependent round trips at the end of every workgroup - n = 4096, k = 14336, 8 rows:
  // 15.6-17.0 us against 10.5 us.)
  float* partial;
  uint32_t kt_per_part;
  // grouped form, gate_up GEMM with silu*mul in the epilogue: the workgroup's first NT/2 column tiles are gate tiles
  // g0.., the other NT/2 the up tiles pair_tiles + g0.. (pair_tiles = inter/16), and out[s, c] = T(silu(T(gate)) * T(up))
  // is [numel, N/2].  0: plain GEMM.
  uint32_t pair_tiles;
  uint32_t x_bytes;  // extent of x, below 1 GiB
  uint32_t nibble_mask, magic2;  // 0x000f000f and T::kMagic2, passed in so that they live in registers
  // Grouped form for a handful of slots (sorted_ids == nullptr): no aligned permutation, expert_ids holds the router's
  // ids [numel] as they are.  Block b is slot b alone: row b / top_k of x, expert expert_ids[b], output row b; an id
  // outside [0, num_experts) leaves its row unwritten, as the alignment would have dropped the slot.
  // TOKSUM instances (the second GEMM with the sum over top-k in it): block b is token b.  Its top_k rows of x
  // [numel, kt_per_expert * 128] lie one behind the other, one row of K = top_k * kt_per_expert * 128 values; k-tile kt
  // of that row meets k-tile kt % kt_per_expert of expert expert_ids[b * top_k + kt / kt_per_expert], its scale times
  // the routing weight topk_w[b * top_k + kt / kt_per_expert]; the fp32 sum over all of K is output row b of [tokens, N].
  uint32_t num_experts;
  uint32_t kt_per_expert;
};

// Eight codes of a packed dword -> MFMA operand holding magic+code (nibble i and i+4 are the pair k=2i, 2i+1).
// mask (0x000f000f) and magic2 arrive as kernel arguments rather than literals: with both in registers the
// compiler folds each and/or pair into one v_and_or_b32, which a literal operand would forbid on this ISA.
template <typename T>
__device__ __forceinline__ typename T::frag dequant_magic_fast(uint32_t w, uint32_t mask, uint32_t magic2) {
  u32x4 v;
  v.x = (w & mask) | magic2;
  v.y = ((w >> 4) & mask) | magic2;
  v.z = ((w >> 8) & mask) | magic2;
  v.w = ((w >> 12) & mask) | magic2;
  return as_frag<T>(v);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// Geometry of the x staging through LDS (XC > 0): the workgroup walks K in chunks of XC k-tiles; the rows of x of one
// chunk lie in LDS as [row][XC * 256 bytes + 64 bytes of padding] (the padding spreads the sixteen rows that one
// fragment read touches over all banks), two chunks deep.  The same LDS holds the cross-wavefront reduction at the end.
template <int MT, int NT, int WAVES, int XC, int XR = 16 * MT>
struct SplitKLds {
  static constexpr int kRows = XR;  // rows of x that are staged: 16 * MT, or fewer when the caller has at most that many
  static constexpr int kRowStride = XC * 256 + 64;
  static constexpr int kChunkBytes = kRows * kRowStride;
  static constexpr int kRedBytes = WAVES * NT * MT * 1024;
  static constexpr int kBytes = (XC > 0 && 2 * kChunkBytes > kRedBytes) ? 2 * kChunkBytes : kRedBytes;
};

// XC == 0: the x fragments travel through registers, in the same ring as the weights (any group size).
// XC > 0 (group 128): x is staged through LDS a chunk of XC k-tiles at a time, each row of a chunk fetched with
// LDS-targeted loads of 1 KiB contiguous bytes; the MFMA fragments are read back from LDS.  That takes the x loads out
// of the ring (16 * MT registers per slot), turns them from 64-byte pieces of sixteen rows into whole cache lines, and
// leaves rows beyond M unfetched.
template <typename T, int MT, int NT, int WAVES, int LOOK, int OCC, int GROUP, bool HAS_ZP, bool GROUPED, int XC = 0,
          int XR = 16 * MT, bool TOKSUM = false>
__global__ void __launch_bounds__(WAVES * 64, OCC) w4a16_splitk_kernel(SplitKParams p) {
  static_assert(!TOKSUM || (GROUPED && MT == 1 && XC == 0 && !HAS_ZP && GROUP == 128), "the token-sum form is a grouped decode form");
  constexpr int GPT = 128 / GROUP;  // groups per k-tile
  constexpr int SPG = GROUP / 32;   // MFMA k-steps per group
  constexpr bool XLDS = XC > 0;
  typedef SplitKLds<MT, NT, WAVES, XC, XR> Lds;
  constexpr int CI = XLDS ? XC / WAVES : 1;                         // rounds per chunk
  constexpr int ND = XLDS ? Lds::kRows * (XC / 4) / WAVES : 0;      // LDS-targeted loads per wavefront and chunk
  constexpr int NW = NT * (1 + GPT * (HAS_ZP ? 2 : 1));             // loads of one ring slot (NT weight tiles)
  static_assert(!XLDS || (GROUP == 128 && XC % 4 == 0 && XC % WAVES == 0 && CI % LOOK == 0 &&
                          (Lds::kRows * (XC / 4)) % WAVES == 0 && LOOK * NW < 64),
                "chunk geometry: whole rounds per chunk, whole ring turns per chunk, equal loads per wavefront");
  const int lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lrow = lane & 15;
  const int lq = lane >> 4;
  const uint32_t KT = TOKSUM ? p.kt_per_expert : p.K / 128;  // k-tiles of a weight strip
  const uint32_t KTL = p.K / 128;                            // k-tiles of a row of x
  const uint32_t G = KT * GPT;
  const bool fused = GROUPED && NT > 1 && p.pair_tiles != 0;
  const uint32_t nt0 = fused ? blockIdx.x * (NT / 2) : blockIdx.x * NT;
  // tiles skipped between the workgroup's column tile NT/2-1 and its column tile NT/2 (0 unless fused)
  const uint32_t pair_extra = fused ? p.pair_tiles - NT / 2 : 0;

  extern __shared__ __attribute__((aligned(16))) char smem[];  // SplitKLds::kBytes
  f32x4 (*red)[NT * MT][64] = reinterpret_cast<f32x4 (*)[NT * MT][64]>(smem);

  // ---- rows of x this lane feeds (row operand: lane l supplies row l%16, k = 8*(l/16)..+7 of each k-step).  A lane
  // whose row lies past M (or is a pad slot) gets an offset beyond the extent of x's buffer resource: its loads fetch
  // nothing and return zero, and its MFMA output rows, which depend on no other row, are never stored.
  constexpr uint32_t kNoRow = 0xffffffffu;
  uint32_t xrow[MT];
  size_t tile_base = 0;  // first weight tile of the expert, in tiles
  size_t sz_base = 0;    // first scale / zero element of the expert
  const bool few = GROUPED && p.sorted_ids == nullptr;  // a handful of slots: one per block, no aligned permutation
  __shared__ uint32_t tok_ids[TOKSUM ? 32 : 1];          // token-sum form: the token's expert ids and routing weights
  __shared__ float tok_w[TOKSUM ? 32 : 1];
  if (GROUPED) {
    const uint32_t pos0 = blockIdx.y * (16 * MT);
    uint32_t e = 0;
    if (TOKSUM) {
      if (threadIdx.x < p.top_k) {
        tok_ids[threadIdx.x] = static_cast<uint32_t>(p.expert_ids[blockIdx.y * p.top_k + threadIdx.x]);
        tok_w[threadIdx.x] = p.topk_w ? p.topk_w[blockIdx.y * p.top_k + threadIdx.x] : 1.0f;
      }
      __syncthreads();
    } else {
      if (!few && pos0 >= static_cast<uint32_t>(p.num_post_pad[0])) return;
      e = static_cast<uint32_t>(p.expert_ids[blockIdx.y]);
      if (few && e >= p.num_experts) return;
    }
    tile_base = static_cast<size_t>(e) * (p.N / 16) * KT;
    sz_base = static_cast<size_t>(e) * G * p.N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if (few || TOKSUM) {
        xrow[mt] = (mt == 0 && lrow == 0) ? (TOKSUM ? blockIdx.y : blockIdx.y / p.top_k) : kNoRow;
      } else {
        const uint32_t sid = static_cast<uint32_t>(p.sorted_ids[pos0 + mt * 16 + lrow]);
        xrow[mt] = sid < p.numel ? sid / p.top_k : kNoRow;
      }
    }
  } else {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const uint32_t r = blockIdx.y * (16 * MT) + mt * 16 + lrow;
      xrow[mt] = r < p.M ? r : kNoRow;
    }
  }

  // ---- buffer resources: bases are wavefront-uniform, lanes add a fixed offset, k-tiles a scalar offset
  const uint32_t w_tile_stride = KT * 1024;  // bytes between consecutive column tiles
  const uint32_t s_tile_stride = G * 32;
  const uint32_t z_tile_stride = G * 16;
  const __amdgpu_buffer_rsrc_t wr = make_rsrc(
      static_cast<const char*>(p.w) + (tile_base + static_cast<size_t>(nt0) * KT) * 1024, (NT + pair_extra) * w_tile_stride);
  const __amdgpu_buffer_rsrc_t sr = make_rsrc(
      static_cast<const char*>(p.scales) + (sz_base + static_cast<size_t>(nt0) * G * 16) * 2, (NT + pair_extra) * s_tile_stride);
  const __amdgpu_buffer_rsrc_t zr = make_rsrc(
      HAS_ZP ? static_cast<const char*>(p.zeros) + sz_base + static_cast<size_t>(nt0) * G * 16 : nullptr,
      HAS_ZP ? (NT + pair_extra) * z_tile_stride : 0);
  const uint32_t pair_w = pair_extra * w_tile_stride, pair_s = pair_extra * s_tile_stride, pair_z = pair_extra * z_tile_stride;
  // x spans less than 1 GiB (checked on the host), so offset kOutOfRange is past this constant extent
  const __amdgpu_buffer_rsrc_t xr = make_rsrc(p.x, 0x3fffffffu);
  const uint32_t w_off = lane * 16;
  const uint32_t s_off = lrow * 2;
  const uint32_t z_off = lrow;
  uint32_t x_off[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) x_off[mt] = xrow[mt] != kNoRow ? (xrow[mt] * p.K + lq * 8) * 2 : 0x40000000u;

  // acc[t][mt][i]: column (nt0+t)*16 + lrow, row mt*16 + 4*lq + i
  f32x4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct Slot {  // one weight tile with its scales / zero points
    u32x4 wq;
    uint32_t sc[GPT];  // 16-bit scale and 8-bit zero point, each widened into a register of its own so that no
    uint32_t zp[GPT];  // packing of ring slots ties loads of different groups together
    float rw;          // token-sum form: the routing weight of the expert this k-tile belongs to
  };
  struct XBuf {
    u32x4 xf[MT][4];
  };
  // Scalar byte offsets of one k-tile in the four buffers.  A k-tile past the end of K gets kOutOfRange:
  // buffer loads beyond the resource's extent return zero, zero x and zero scales contribute nothing, and every
  // wavefront runs the same instruction sequence, so the waits count exactly the loads allowed to stay in flight.
  constexpr uint32_t kOutOfRange = 0x40000000u;
  struct KOff {
    uint32_t w, s, z, x;
    __amdgpu_buffer_rsrc_t wr, sr;  // token-sum form: the weights and scales of the k-tile's expert
    float rw;
  };
  const uint32_t kt_begin = GROUPED ? 0 : blockIdx.z * p.kt_per_part;
  const uint32_t kt_end = GROUPED ? KTL : ((KTL - kt_begin) < p.kt_per_part ? KTL : kt_begin + p.kt_per_part);
  auto koff = [&](uint32_t round) {
    const uint32_t kt = kt_begin + wave + round * WAVES;
    bool ok = kt < kt_end;
    KOff o;
    uint32_t ktw = kt;  // k-tile inside the weight strip
    if constexpr (TOKSUM) {
      // which expert's strip this k-tile of the token's row meets: a resource of its own per expert (the stack of all
      // experts is larger than one resource's offsets may span)
      const uint32_t j = ok ? kt / KT : 0;
      ktw = kt - j * KT;
      const uint32_t e = __builtin_amdgcn_readfirstlane(tok_ids[j]);
      o.rw = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, tok_w[j])));
      ok = ok && e < p.num_experts;
      const size_t e_ok = e < p.num_experts ? e : 0;
      o.wr = make_rsrc(static_cast<const char*>(p.w) + ((e_ok * (p.N / 16) + nt0) * KT) * 1024, NT * w_tile_stride);
      o.sr = make_rsrc(static_cast<const char*>(p.scales) + (e_ok * G * p.N + static_cast<size_t>(nt0) * G * 16) * 2, NT * s_tile_stride);
    }
    // readfirstlane pins the offsets to scalar registers (a vector offset would make every load a waterfall loop)
    o.w = __builtin_amdgcn_readfirstlane(ok ? ktw * 1024u : kOutOfRange);
    o.s = __builtin_amdgcn_readfirstlane(ok ? ktw * (GPT * 32u) : kOutOfRange);
    o.z = __builtin_amdgcn_readfirstlane(ok ? ktw * (GPT * 16u) : kOutOfRange);
    o.x = __builtin_amdgcn_readfirstlane(ok ? kt * 256u : kOutOfRange);
    return o;
  };

  auto load_slot = [&](Slot& s, int t, const KOff& o) {
    const bool upper = NT > 1 && t >= NT / 2;  // the up tiles of a fused gate_up workgroup lie pair_extra tiles further
    if constexpr (TOKSUM) {
      s.wq = __builtin_amdgcn_raw_buffer_load_b128(o.wr, w_off, t * w_tile_stride + o.w, 2);
      s.sc[0] = __builtin_amdgcn_raw_buffer_load_b16(o.sr, s_off, t * s_tile_stride + o.s, 0);
      s.rw = o.rw;
      return;
    }
    s.wq = __builtin_amdgcn_raw_buffer_load_b128(wr, w_off, t * w_tile_stride + (upper ? pair_w : 0) + o.w, 2);
#pragma unroll
    for (int gi = 0; gi < GPT; ++gi) {
      s.sc[gi] = __builtin_amdgcn_raw_buffer_load_b16(sr, s_off, t * s_tile_stride + (upper ? pair_s : 0) + o.s + gi * 32, 0);
      if (HAS_ZP) s.zp[gi] = __builtin_amdgcn_raw_buffer_load_b8(zr, z_off, t * z_tile_stride + (upper ? pair_z : 0) + o.z + gi * 16, 0);
    }
  };
  auto load_x = [&](XBuf& b, const KOff& o) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int d = 0; d < 4; ++d) b.xf[mt][d] = __builtin_amdgcn_raw_buffer_load_b128(xr, x_off[mt], o.x + d * 64, 0);
  };

  // The operand of the sum-of-x MFMA: ones with zero points (the sum is then multiplied by each column's own offset);
  // without them the offset is the same -(magic + 8) for every column, so the MFMA multiplies by it directly and its
  // result is what the weight MFMAs of the group start from: r = -(magic + 8) * sum(x) + sum((magic + code) * x).
  constexpr uint32_t kSumOperand = HAS_ZP ? T::kOne2 : T::kNegSym2;
  const typename T::frag ones = as_frag<T>(u32x4{kSumOperand, kSumOperand, kSumOperand, kSumOperand});
  uint32_t magic2 = p.magic2;
  asm volatile("" : "+v"(magic2));  // no instruction: keeps the value in a VGPR so the three-operand form applies
  const uint32_t nmask = p.nibble_mask;

  // LIVE: the row tiles that are multiplied (all MT, or one of two when the block's second row tile holds no row)
  auto sum_x = [&](auto live_c, const XBuf& b, f32x4 (&sx)[GPT][MT]) {
    constexpr int LIVE = decltype(live_c)::value;
#pragma unroll
    for (int gi = 0; gi < GPT; ++gi)
#pragma unroll
      for (int mt = 0; mt < LIVE; ++mt) {
        f32x4 r{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = gi * SPG; d < (gi + 1) * SPG; ++d) r = T::mfma(as_frag<T>(b.xf[mt][d]), ones, r);
        sx[gi][mt] = r;
      }
  };
  auto compute = [&](auto live_c, const Slot& s, const XBuf& b, const f32x4 (&sx)[GPT][MT], int t) {
    constexpr int LIVE = decltype(live_c)::value;
#pragma unroll
    for (int gi = 0; gi < GPT; ++gi) {
      const float sc = TOKSUM ? T::lo_to_float(s.sc[gi]) * s.rw : T::lo_to_float(s.sc[gi]);
      const float ncz = HAS_ZP ? -(T::kMagic + static_cast<float>(s.zp[gi])) : -(T::kMagic + 8.0f);
      typename T::frag wf[SPG];
#pragma unroll
      for (int d = 0; d < SPG; ++d) wf[d] = dequant_magic_fast<T>(s.wq[gi * SPG + d], nmask, magic2);
#pragma unroll
      for (int mt = 0; mt < LIVE; ++mt) {
        f32x4 r = HAS_ZP ? f32x4{0.f, 0.f, 0.f, 0.f} : sx[gi][mt];
#pragma unroll
        for (int d = 0; d < SPG; ++d) r = T::mfma(as_frag<T>(b.xf[mt][gi * SPG + d]), wf[d], r);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[t][mt][i] = HAS_ZP ? __builtin_fmaf(sc, __builtin_fmaf(ncz, sx[gi][mt][i], r[i]), acc[t][mt][i])
                                 : __builtin_fmaf(sc, r[i], acc[t][mt][i]);
      }
    }
  };

  // ---- main loop.  The ring holds LOOK k-tiles, each a load group of NT weight tiles (with scales / zero points)
  // followed, in the register form, by the x fragments; a group is refilled for round cur+LOOK while round cur is
  // consumed, so LOOK-1 whole groups stay in flight behind every wait.  The round count is uniform over the workgroup
  // and a multiple of LOOK (of the rounds of a chunk in the LDS form), the surplus rounds load zeros.
  // The main loop exists once per number of row tiles that are multiplied.  A 32-row expert block whose second row
  // tile holds no slot (an expert with at most 16 rows: at 16 rows per expert on average, every second one) runs the
  // loop over one row tile: the MFMAs, sum-of-x MFMAs and scale FMAs of the empty tile are what puts the two-tile form
  // over a SIMD's issue slots.  The choice is made once per workgroup, outside the loop.
  bool second_empty = false;
  if constexpr (GROUPED && MT == 2) second_empty = __builtin_amdgcn_ballot_w64(xrow[1] != kNoRow) == 0;
  auto run_live = [&](auto&& loop) {
    if constexpr (GROUPED && MT == 2) {
      if (second_empty)
        loop(std::integral_constant<int, 1>{});
      else
        loop(std::integral_constant<int, 2>{});
    } else {
      loop(std::integral_constant<int, MT>{});
    }
  };
  const uint32_t slice_len = kt_end - kt_begin;
  Slot slot[LOOK][NT];
  if constexpr (!XLDS) {
    const uint32_t rounds = (slice_len + WAVES * LOOK - 1) / (WAVES * LOOK) * LOOK;
    XBuf xb[LOOK];
#pragma unroll
    for (int j = 0; j < LOOK; ++j) {
      const KOff o = koff(j);
#pragma unroll
      for (int t = 0; t < NT; ++t) load_slot(slot[j][t], t, o);
      load_x(xb[j], o);
      __builtin_amdgcn_sched_barrier(0);  // keep the groups in issue order, the waits below count on it
    }
    auto loop = [&](auto live_c) {
    for (uint32_t it = 0; it < rounds; it += LOOK) {
#pragma unroll
      for (int h = 0; h < LOOK; ++h) {
        const KOff o = koff(it + h + LOOK);  // past the last round this is out of range by construction
        f32x4 sx[GPT][MT];
        sum_x(live_c, xb[h], sx);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          compute(live_c, slot[h][t], xb[h], sx, t);
          // the refill must be issued here, not sunk below the remaining math: the barriers pin it in place
          __builtin_amdgcn_sched_barrier(0);
          load_slot(slot[h][t], t, o);
          __builtin_amdgcn_sched_barrier(0);
        }
        load_x(xb[h], o);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    };
    run_live(loop);
  } else {
    // Rows of the block that hold data (they come first: pad slots of an expert's block lie at its end).
    uint32_t nrows;
    if (GROUPED) {
      nrows = 0;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        nrows += static_cast<uint32_t>(__builtin_popcountll(__builtin_amdgcn_ballot_w64(lq == 0 && xrow[mt] != kNoRow)));
      nrows = __builtin_amdgcn_readfirstlane(nrows);
    } else {
      const uint32_t left = p.M - blockIdx.y * (16 * MT);
      nrows = left < static_cast<uint32_t>(Lds::kRows) ? left : static_cast<uint32_t>(Lds::kRows);
    }
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char*)smem));
    const uint32_t nchunks = (slice_len + XC - 1) / XC;
    // Chunk c -> LDS buffer c % 2.  Wavefront w issues loads w, w + WAVES, ... of the chunk's kRows * XC/4 loads; load
    // (r, q) moves k-tiles 4q..4q+3 of row r, 1 KiB contiguous (lane j: bytes 16j..16j+15).  Lanes past the end of the row
    // (K/128 not a multiple of 4) re-read its start: finite values, multiplied by weights that were loaded as zero.
    // Loads of rows that hold no data, or of k-tile groups past the range, are skipped: the counts the waits below
    // rely on do not include these loads.
    auto stage_chunk = [&](uint32_t c) {
      const uint32_t kt0 = c * XC;
#pragma unroll
      for (int i = 0; i < ND; ++i) {
        const uint32_t idx = wave + i * WAVES;
        const uint32_t r = idx / (XC / 4), q = idx % (XC / 4);
        if (r < nrows && kt0 + 4 * q < slice_len) {
          uint32_t src_row;
          if (GROUPED) {
            const uint32_t v = (MT > 1 && r >= 16) ? xrow[MT - 1] : xrow[0];
            src_row = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), static_cast<int>(r & 15u)));
          } else {
            src_row = blockIdx.y * (16 * MT) + r;
          }
          const uint32_t kt_abs = kt_begin + kt0 + 4 * q;
          const char* src = static_cast<const char*>(p.x) + (static_cast<size_t>(src_row) * p.K + static_cast<size_t>(kt_abs) * 128) * 2;
          const uint32_t left_bytes = (KT - kt_abs) * 256u;  // of the row, from this group's first byte
          const uint32_t voff = static_cast<uint32_t>(lane) * 16u < left_bytes ? static_cast<uint32_t>(lane) * 16u : 0u;
          const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + (c & 1u) * Lds::kChunkBytes + r * Lds::kRowStride + q * 1024u);
          // (s_nop 4: scalar operands that a v_readfirstlane produced need five wait states before a vector memory
          // instruction reads them, and the compiler inserts none inside an assembly statement.  M0 is named as
          // clobbered; the compiler treats it as a reserved register and keeps no value of its own in it across
          // statements - it writes M0 right in front of each instruction of its own that reads it.)
          asm volatile("s_nop 4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %2"
                       :
                       : "v"(voff), "s"(dst), "s"(src)
                       : "memory", "m0");
        }
      }
    };
    // fragments of local k-tile `lk` of chunk c: lane (row, quarter) reads 16 bytes of each of the four k-steps
    auto read_x = [&](XBuf& b, uint32_t c, uint32_t lk) {
      const char* base = smem + (c & 1u) * Lds::kChunkBytes + lk * 256u + lq * 16;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int d = 0; d < 4; ++d)
          b.xf[mt][d] = *reinterpret_cast<const u32x4*>(base + ((mt * 16 + lrow) % XR) * Lds::kRowStride + d * 64);
    };
    // wait until at most LOOK ring slots' loads are outstanding.  Every staging load of the next chunk was issued
    // before the CI >= LOOK refills of this chunk, and loads retire in issue order: the chunk has landed.
    auto wait_staged = [&]() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOOK * NW) : "memory"); };

    stage_chunk(0);
#pragma unroll
    for (int j = 0; j < LOOK; ++j) {
      const KOff o = koff(j);
#pragma unroll
      for (int t = 0; t < NT; ++t) load_slot(slot[j][t], t, o);
      __builtin_amdgcn_sched_barrier(0);
    }
    wait_staged();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");  // no LDS read may move above the barrier
    auto loop = [&](auto live_c) {
    for (uint32_t c = 0; c < nchunks; ++c) {
      if (c + 1 < nchunks) stage_chunk(c + 1);  // into the buffer chunk c-1 used: every wavefront is past the barrier behind it
#pragma unroll
      for (int j = 0; j < CI; ++j) {
        const int h = j % LOOK;
        const KOff o = koff(c * CI + j + LOOK);
        XBuf xb;
        read_x(xb, c, wave + j * WAVES);
        if (wave + (c * CI + j) * WAVES >= slice_len) {
          // a surplus round: its k-tile was not staged (whatever the LDS holds there need not be finite) and its
          // weights and scales were loaded as zero
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int d = 0; d < 4; ++d) xb.xf[mt][d] = u32x4{0u, 0u, 0u, 0u};
        }
        f32x4 sx[GPT][MT];
        sum_x(live_c, xb, sx);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          compute(live_c, slot[h][t], xb, sx, t);
          __builtin_amdgcn_sched_barrier(0);
          load_slot(slot[h][t], t, o);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      wait_staged();
      __builtin_amdgcn_s_barrier();  // chunk c+1 is in LDS for everyone, and everyone is done with chunk c
      asm volatile("" ::: "memory");
    }
    };
    run_live(loop);
  }

  // ---- cross-wavefront reduction in wavefront order
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[wave][t * MT + mt][lane] = acc[t][mt];
  __syncthreads();

  // Grouped form: the slot ids (and routing weights) of the rows this thread stores, fetched before the first store.
  // Read next to each store they would wait for the stores in front of them - the compiler cannot know that the output
  // does not overlap the index arrays - one memory round trip after the other.
  static_assert(MT <= 2, "the epilogue selects between two row tiles");
  u32x4 esid[MT];
  f32x4 erw[MT];
  if (GROUPED) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        esid[mt][i] = (few || TOKSUM) ? ((mt == 0 && 4 * lq + i == 0) ? blockIdx.y : kNoRow)
                                      : static_cast<uint32_t>(p.sorted_ids[blockIdx.y * (16 * MT) + mt * 16 + 4 * lq + i]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        erw[mt][i] = (!TOKSUM && !fused && esid[mt][i] < p.numel && p.topk_w) ? p.topk_w[esid[mt][i]] : 1.0f;
  }

  if (GROUPED && NT > 1 && fused) {
    // gate_up with silu*mul: both sums are rounded to T as the unfused GEMM would store them, then
    // silu(g) * u in fp32 and one more rounding, the arithmetic of silu_mul_kernel
    constexpr int HALF = NT > 1 ? NT / 2 : 1;
    const uint32_t out_n = p.N / 2;
    for (int idx = threadIdx.x; idx < HALF * MT * 64; idx += WAVES * 64) {
      const int l = idx & 63;
      const int tm = idx >> 6;
      const int t = tm / MT, mt = tm % MT;
      f32x4 g = red[0][t * MT + mt][l], u = red[0][(t + HALF) * MT + mt][l];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) {
        g += red[w][t * MT + mt][l];
        u += red[w][(t + HALF) * MT + mt][l];
      }
      const uint32_t col = (nt0 + t) * 16 + (l & 15);
      const u32x4 msid = (MT > 1 && mt) ? esid[MT - 1] : esid[0];  // (a select: no register is indexed)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t sid = msid[i];
        if (sid < p.numel) {
          const float gv = T::to_float(T::from_float(g[i])), uv = T::to_float(T::from_float(u[i]));
          const float y = silu_mul_f32(gv, uv);
          static_cast<uint16_t*>(p.y)[static_cast<size_t>(sid) * out_n + col] = T::from_float(y);
        }
      }
    }
    return;
  }

  const bool cut = !GROUPED && p.partial != nullptr;
  for (int idx = threadIdx.x; idx < NT * MT * 64; idx += WAVES * 64) {
    const int l = idx & 63;
    const int tm = idx >> 6;
    const int t = tm / MT, mt = tm % MT;
    f32x4 v = red[0][tm][l];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) v += red[w][tm][l];
    const uint32_t col = (nt0 + t) * 16 + (l & 15);
    u32x4 msid = {};
    f32x4 mrw = {};
    if (GROUPED) {  // (selects: no register is indexed)
      msid = (MT > 1 && mt) ? esid[MT - 1] : esid[0];
      mrw = (MT > 1 && mt) ? erw[MT - 1] : erw[0];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t r = mt * 16 + 4 * (l >> 4) + i;
      uint32_t orow;
      bool valid;
      float rw = 1.0f;
      if (GROUPED) {
        const uint32_t sid = msid[i];
        valid = sid < p.numel;
        orow = sid;
        rw = mrw[i];
      } else {
        orow = blockIdx.y * (16 * MT) + r;
        valid = orow < p.M;
      }
      if (valid) {
        if (cut)
          p.partial[(static_cast<size_t>(blockIdx.z) * p.M + orow) * p.N + col] = v[i];
        else
          static_cast<uint16_t*>(p.y)[static_cast<size_t>(orow) * p.N + col] = T::from_float(v[i] * rw);
      }
    }
  }
}

}  // namespace ksq
