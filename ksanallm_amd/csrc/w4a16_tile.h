// Prefill-regime W4A16 kernel (MFMA-bound): a workgroup of 8 wavefronts computes a BM x 256 output tile
// (BM = 256 or 128) over all of K or, for tiles that are cut along K (tile_work.h), over a contiguous range of k-tiles.
//
//   - x (activations) goes global -> LDS without touching registers: every wavefront issues global_load_lds_dwordx4
//     for whole 1 KiB MFMA fragments (16 rows x 32 k, four lanes per row so that every load touches 64 contiguous
//     bytes per row, pieces swizzled so that the read-back is free of bank conflicts), into a ring of NS stages of
//     64 k each.  The fragment is read back with one ds_read_b128 per lane, DEPTH fragments ahead of the MFMAs that
//     use it.  Two to three stages are in flight while one is consumed; the one barrier per stage sits in the middle
//     of the stage, so the fragment reads never drain at a stage boundary.
//   - packed int4 weights never touch LDS: the 8 wavefronts split the 256 columns (2 column tiles of 16 each), so
//     every weight fragment belongs to exactly one wavefront and no weight is dequantized twice.  A wavefront loads
//     its 1 KiB tiles straight from global memory (16 bytes per lane) three stages ahead and dequantizes them in
//     registers to T with (code - zp) * s applied.
//   - the loads of a stage are not issued in one run behind the barrier - eight wavefronts would queue at the memory
//     pipeline at once, each stalled until its loads are accepted - but one group at a time between the MFMAs of the
//     steps: x fragments during the second step of every stage, weights during the first step of every other one.
//   - all vector memory loads of the main loop are issued from inline assembly in a fixed order, the same number
//     every stage (addresses are clamped past the end), so that one `s_waitcnt vmcnt(N)` per stage with a constant N
//     releases exactly the stage that is needed: vmcnt retires in issue order.  The registers a wait makes valid are
//     tied to that wait as in/out operands, which keeps the compiler from scheduling their uses above it.
//   - the weights are the row operand of v_mfma_f32_16x16x32 and x the column operand, so a lane ends up with four
//     consecutive output columns of one row and stores them as one 8-byte word (or 16 bytes of fp32 partials).
//
// Workgroup ids are remapped (tile_work.h) so that the workgroups running on one XCD at the same time form a compact
// block of row tiles x column tiles: both operands are then shared through that XCD's L2.
#pragma once

#include <type_traits>

#include "ksq_common.h"
#include "tile_work.h"
#include "splitk_reduce.h"

namespace ksq {

struct TileParams {
  void* y;
  const void* x;
  const void* w;
  const void* scales;
  const void* zeros;
  float* partial;  // [slot][part][BM][256] fp32 tiles of the workgroups that compute a part of K
  float* y32;      // dense form, verification only: the fp32 sums go here, [M, N], and nothing is rounded to T
  uint32_t M, N, K;
  uint32_t tiles_m, tiles_n;
  uint32_t main_items, splits, kt_per_split;  // tile_work.h
  // grouped (MoE) form: row block b = tile_m holds the rows sorted_ids[b*BM ..] of expert expert_ids[b]
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_w;  // optional: multiplied into the output row of slot id s
  uint32_t numel, top_k;
  // grouped form, gate_up weights with silu(gate) * up in the epilogue: a wavefront's second column tile is the up tile
  // pair_tiles (= N / 32) column tiles behind its gate tile, a workgroup covers 128 gate columns and the output has
  // N / 2 columns.  0: plain GEMM.
  uint32_t pair_tiles;
};

// dequantize one packed dword (8 codes) to 8 T values with (code - zp) * s applied
template <typename T, bool HAS_ZP>
struct Dequant;

// fp16: 0x6400 | code is the half 1024 + code, and a nibble left in bits 4..7 gives 1024 + 16*code, which saves the
// shifts of the odd nibbles.  code - zp is formed exactly ((1024+code) - (1024+zp), or (1024+16 code)/16 - (64+zp)),
// then multiplied by the scale: one rounding per weight.
template <bool HAS_ZP>
struct Dequant<F16, HAS_ZP> {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  h2 s2, c1, c16;  // (s,s), 1024+zp, 64+zp : the zero point is removed exactly in integers before the scale
  __device__ __forceinline__ void set(uint32_t scale_bits, uint32_t zp) {
    const _Float16 s = __builtin_bit_cast(_Float16, static_cast<uint16_t>(scale_bits));
    const float z = HAS_ZP ? static_cast<float>(zp) : 8.0f;
    s2 = h2{s, s};
    const _Float16 a = static_cast<_Float16>(1024.0f + z), b = static_cast<_Float16>(64.0f + z);
    c1 = h2{a, a};
    c16 = h2{b, b};
  }
  __device__ __forceinline__ F16::frag operator()(uint32_t w) const {
    const h2 sixteenth{static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
    // (x & mask) | magic in one instruction: on this ISA the three-operand form takes no literal, so the mask comes
    // from a scalar register and the magic from a vector register
    const uint32_t magic = 0x64006400u;
    const uint32_t w8 = w >> 8;
    uint32_t lo0, hi0, lo1, hi1;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(lo0) : "v"(w), "s"(0x000f000fu), "v"(magic));   // k = 0,1 : 1024 + code
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(hi0) : "v"(w), "s"(0x00f000f0u), "v"(magic));   // k = 2,3 : 1024 + 16*code
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(lo1) : "v"(w8), "s"(0x000f000fu), "v"(magic));  // k = 4,5
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(hi1) : "v"(w8), "s"(0x00f000f0u), "v"(magic));  // k = 6,7
    h2 r0 = (__builtin_bit_cast(h2, lo0) - c1) * s2;
    h2 r1 = (__builtin_bit_cast(h2, hi0) * sixteenth - c16) * s2;
    h2 r2 = (__builtin_bit_cast(h2, lo1) - c1) * s2;
    h2 r3 = (__builtin_bit_cast(h2, hi1) * sixteenth - c16) * s2;
    u32x4 v{__builtin_bit_cast(uint32_t, r0), __builtin_bit_cast(uint32_t, r1), __builtin_bit_cast(uint32_t, r2),
            __builtin_bit_cast(uint32_t, r3)};
    return as_frag<F16>(v);
  }
};

// bf16 has no packed arithmetic on this ISA: codes go through fp32 and are packed back with v_cvt_pk_bf16_f32.  A byte
// 0x0u (u = 0..15) read as OCP e4m3 is exactly u * 2^-9 (the subnormal range), so one v_cvt_pk_f32_fp8 turns two codes
// into floats; 2^9 is folded into the scale (exact), and fma(u * 2^-9, s * 2^9, -zp * s) is the same real number rounded
// once as fma(u, s, -zp * s).  19 instructions per packed dword (2 masks and a shift, 4 conversions, 8 fmas, 4 packs).
template <bool HAS_ZP>
struct Dequant<BF16, HAS_ZP> {
  float s, b;  // s * 2^9 and -zp*s
  __device__ __forceinline__ void set(uint32_t scale_bits, uint32_t zp) {
    const float sc = BF16::lo_to_float(scale_bits);
    b = -(HAS_ZP ? static_cast<float>(zp) : 8.0f) * sc;
    s = sc * 512.0f;
  }
  static __device__ __forceinline__ uint32_t pk(float a, float c) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    b2 r = __builtin_convertvector(f2{a, c}, b2);
    return __builtin_bit_cast(uint32_t, r);
  }
  __device__ __forceinline__ BF16::frag operator()(uint32_t w) const {
    typedef float f2 __attribute__((ext_vector_type(2)));
    // nibble p holds k = {0,2,4,6,1,3,5,7}[p]: even nibbles p=0,2,4,6 -> k=0,4,1,5 ; odd p=1,3,5,7 -> k=2,6,3,7
    const uint32_t e = w & 0x0f0f0f0fu;
    const uint32_t o = (w >> 4) & 0x0f0f0f0fu;
    const f2 k04 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(e), false);
    const f2 k15 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(e), true);
    const f2 k26 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(o), false);
    const f2 k37 = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(o), true);
    u32x4 v;
    v.x = pk(__builtin_fmaf(k04[0], s, b), __builtin_fmaf(k15[0], s, b));
    v.y = pk(__builtin_fmaf(k26[0], s, b), __builtin_fmaf(k37[0], s, b));
    v.z = pk(__builtin_fmaf(k04[1], s, b), __builtin_fmaf(k15[1], s, b));
    v.w = pk(__builtin_fmaf(k26[1], s, b), __builtin_fmaf(k37[1], s, b));
    return as_frag<BF16>(v);
  }
};

// One column tile's packed weights for one k-tile of 128, with the scale and zero point of each of its GPT groups.
template <int GPT>
struct WSlot {
  u32x4 wq;
  uint32_t sc[GPT];
  uint32_t zp[GPT];
};

// 8 wavefronts side by side along N; each computes WM x 2 tiles of 16x16.  BM = 16*WM, BN = 256.
// GROUPED: the MoE form.  Row block tile_m is one block of the aligned token permutation: its rows are gathered through
// sorted_ids (slot id s reads x row s / top_k, pad slots carry s >= numel), its weights are those of expert
// expert_ids[tile_m], its results are scattered to out[s, :] (times topk_w[s] when given).  Blocks past num_post_pad
// leave at once.  There is no split-K in this form.
// GROUP: rows of a quantization group, 128, 64 or 32 (GPT = 128 / GROUP groups per k-tile).
template <typename T, int WM, bool HAS_ZP, bool GROUPED = false, int GROUP = 128>
__global__ void __launch_bounds__(512, 1) w4a16_tile_kernel(TileParams p) {
  static_assert(GROUP == 128 || GROUP == 64 || GROUP == 32, "group size");
  constexpr int GPT = 128 / GROUP;
  typedef ksq::WSlot<GPT> WSlot;
  constexpr int WAVES = 8;
  constexpr int WN = 2;
  constexpr int BM = WM * 16;
  constexpr int BN = WAVES * WN * 16;
  constexpr int BK = 64;                 // k per LDS stage
  constexpr int NS = 4;                  // LDS stages
  constexpr int FRAGS = WM * (BK / 32);  // 1 KiB fragments per stage
  constexpr int STAGE_BYTES = FRAGS * 1024;
  constexpr int AP = FRAGS / WAVES;      // fragments this wavefront fetches per stage
  constexpr int WL = 1 + GPT * (HAS_ZP ? 2 : 1);  // loads per weight slot: the tile, and a scale (and zero point) per group
  constexpr int L = WL + AP;             // vector memory loads per wavefront per stage
  constexpr int WAIT_N = (NS - 2) * L;   // loads issued after the stage that is about to be consumed
  static_assert(FRAGS % WAVES == 0 && AP % 2 == 0, "fragments must split evenly, in k pairs, over the wavefronts");
  static_assert(WAIT_N < 64, "vmcnt is a 6-bit counter");

  extern __shared__ __attribute__((aligned(16))) char lds[];  // NS * STAGE_BYTES

  const int lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lrow = lane & 15, lq = lane >> 4;
  const uint32_t KT = p.K / 128;

  // ---- work id (tile_work.h): output tile and the part of K this workgroup computes
  // (the divisions inside run on the vector unit: readfirstlane brings the wave-uniform results back to scalars)
  const TileWork work = tile_work(blockIdx.x, p.tiles_m, p.tiles_n, p.main_items, p.splits, GROUPED);
  const uint32_t tile_m = __builtin_amdgcn_readfirstlane(work.tile_m), tile_n = __builtin_amdgcn_readfirstlane(work.tile_n);
  const uint32_t part = __builtin_amdgcn_readfirstlane(work.part), slot = __builtin_amdgcn_readfirstlane(work.slot);
  const bool direct = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(work.direct)) != 0;
  const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
  const uint32_t kt_begin = direct ? 0 : part * p.kt_per_split;
  const uint32_t kt_count = direct ? KT : ((KT - kt_begin) < p.kt_per_split ? (KT - kt_begin) : p.kt_per_split);
  const uint32_t stages = kt_count * 2;
  uint32_t expert = 0;
  // Row tiles (16 rows) of this block that hold rows at all: the last row block of the matrix may be short, and in the
  // grouped form an expert's last block is padded to the block size with the pad slots at its end.
  uint32_t live_tiles = WM;
  if (!GROUPED) {
    const uint32_t rows = p.M - m0;
    live_tiles = rows < static_cast<uint32_t>(BM) ? (rows + 15) / 16 : WM;
  }
  if (GROUPED) {
    if (m0 >= static_cast<uint32_t>(p.num_post_pad[0])) return;  // uniform: the whole workgroup leaves
    expert = static_cast<uint32_t>(p.expert_ids[tile_m]);
    uint32_t rows = 0;
#pragma unroll
    for (int h = 0; h < BM / 64; ++h) {
      const bool is_row = static_cast<uint32_t>(p.sorted_ids[m0 + h * 64 + lane]) < p.numel;
      rows += static_cast<uint32_t>(__builtin_popcountll(__builtin_amdgcn_ballot_w64(is_row)));
    }
    live_tiles = __builtin_amdgcn_readfirstlane((rows + 15) / 16);
  }

  // ---- x staging: this wavefront fetches fragments f = wave*AP + 2j + {0,1}: row block f/2, k half f%2.
  // A fragment (16 rows x 32 k = 64 bytes per row) is fetched by ONE load in which four consecutive lanes take the
  // four 16-byte pieces of one row - 64 contiguous bytes, the granularity at which the memory pipeline runs at full
  // rate (16-byte pieces of four different rows run at a quarter of it).  Load lane j lands at 16*j = 64*(j/4) +
  // 16*(j%4); it fetches piece (j%4) ^ (j/16) of row j/4, so that MFMA lane (row r, k piece q) finds its operand at
  // 64*r + 16*(q ^ (r/4)): the sixteen lanes that read together (same q) then hit sixteen different bank groups.
  const char* x_tile = static_cast<const char*>(p.x) + (static_cast<size_t>(GROUPED ? 0 : m0) * p.K + kt_begin * 128) * 2;
  const uint32_t a_rd = 64 * lrow + 16 * (lq ^ (lrow >> 2));  // this lane's operand inside a fragment
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char*)lds));

  // ---- weights: this wavefront's two column tiles (clamped inside N; results of clamped tiles are not stored)
  const uint32_t n_tiles = p.N / 16;
  const bool paired = GROUPED && p.pair_tiles != 0;
  const uint32_t nt0 = paired ? tile_n * WAVES + wave : n0 / 16 + wave * WN;
  const char* w_base[WN];
  const char* s_base[WN];
  const char* z_base[WN];
#pragma unroll
  for (int t = 0; t < WN; ++t) {
    uint32_t col_tile = (nt0 + t < n_tiles) ? nt0 + t : n_tiles - 1;
    if (paired) col_tile = (nt0 < p.pair_tiles ? nt0 : p.pair_tiles - 1) + t * p.pair_tiles;
    const size_t nt = static_cast<size_t>(expert) * n_tiles + col_tile;
    w_base[t] = static_cast<const char*>(p.w) + (nt * KT + kt_begin) * 1024;
    s_base[t] = static_cast<const char*>(p.scales) + (nt * KT + kt_begin) * (GPT * 32);
    z_base[t] = HAS_ZP ? static_cast<const char*>(p.zeros) + (nt * KT + kt_begin) * (GPT * 16) : nullptr;
  }
  const uint32_t w_voff = lane * 16, s_voff = lrow * 2, z_voff = lrow;

  f32x4 acc[WN][WM];
#pragma unroll
  for (int t = 0; t < WN; ++t)
#pragma unroll
    for (int i = 0; i < WM; ++i) acc[t][i] = f32x4{0.f, 0.f, 0.f, 0.f};

  WSlot ring[3][WN];  // k-tiles kt, kt+1, kt+2 (indexed kt % 3)

  // ---- issue helpers (inline assembly: the compiler neither reorders nor counts these loads)
  // Every group of loads is ONE assembly statement that opens with `s_nop 4`: all its scalar operands are in place
  // before the statement starts, and should the compiler have produced one of them with a VALU instruction
  // (v_readfirstlane), the five wait states a vector memory instruction needs after that have passed.  The compiler
  // inserts such wait states for its own instructions, not inside assembly.
  // the loads of one column tile for k-tile kt: the packed tile, and a scale (and zero point) per group
  auto load_w_part = [&](WSlot (&dst)[WN], uint32_t kt, auto tc) {
    constexpr int t = decltype(tc)::value;
    kt = kt < kt_count ? kt : kt_count - 1;
    const char* w0 = w_base[t] + static_cast<size_t>(kt) * 1024;
    const char* s0 = s_base[t] + static_cast<size_t>(kt) * (GPT * 32);
    if (HAS_ZP) {
      const char* z0 = z_base[t] + static_cast<size_t>(kt) * (GPT * 16);
      asm volatile(
          "s_nop 4\n\t"
          "global_load_dwordx4 %0, %3, %6\n\t"
          "global_load_ushort %1, %4, %7\n\t"
          "global_load_ubyte %2, %5, %8"
          : "=&v"(dst[t].wq), "=&v"(dst[t].sc[0]), "=&v"(dst[t].zp[0])
          : "v"(w_voff), "v"(s_voff), "v"(z_voff), "s"(w0), "s"(s0), "s"(z0)
          : "memory");
#pragma unroll
      for (int gi = 1; gi < GPT; ++gi) {
        const char* s0g = s0 + gi * 32;
        const char* z0g = z0 + gi * 16;
        asm volatile(
            "s_nop 4\n\t"
            "global_load_ushort %0, %2, %4\n\t"
            "global_load_ubyte %1, %3, %5"
            : "=&v"(dst[t].sc[gi]), "=&v"(dst[t].zp[gi])
            : "v"(s_voff), "v"(z_voff), "s"(s0g), "s"(z0g)
            : "memory");
      }
    } else {
      asm volatile(
          "s_nop 4\n\t"
          "global_load_dwordx4 %0, %2, %4\n\t"
          "global_load_ushort %1, %3, %5"
          : "=&v"(dst[t].wq), "=&v"(dst[t].sc[0])
          : "v"(w_voff), "v"(s_voff), "s"(w0), "s"(s0)
          : "memory");
#pragma unroll
      for (int gi = 1; gi < GPT; ++gi) {
        const char* s0g = s0 + gi * 32;
        asm volatile("s_nop 4\n\tglobal_load_ushort %0, %1, %2" : "=&v"(dst[t].sc[gi]) : "v"(s_voff), "s"(s0g) : "memory");
      }
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi) dst[t].zp[gi] = 8u;
    }
  };
  auto load_w = [&](WSlot (&dst)[WN], uint32_t kt) {
    static_assert(WN == 2, "two column tiles per wavefront");
    load_w_part(dst, kt, std::integral_constant<int, 0>{});
    load_w_part(dst, kt, std::integral_constant<int, 1>{});
  };
  // wait until at most `n` loads are outstanding; the weight slots named become valid with this wait and are tied to it
  auto wait_tie = [&](auto n, WSlot (&fresh)[WN]) {
    asm volatile("s_waitcnt vmcnt(%6)"
                 : "+v"(fresh[0].wq), "+v"(fresh[0].sc[0]), "+v"(fresh[0].zp[0]), "+v"(fresh[1].wq), "+v"(fresh[1].sc[0]),
                   "+v"(fresh[1].zp[0])
                 : "n"(decltype(n)::value)
                 : "memory");
    // (the further groups' registers became valid with the same wait: an empty statement, which stays behind the wait
    // like every volatile statement, ties them to it)
#pragma unroll
    for (int gi = 1; gi < GPT; ++gi)
      asm volatile("" : "+v"(fresh[0].sc[gi]), "+v"(fresh[0].zp[gi]), "+v"(fresh[1].sc[gi]), "+v"(fresh[1].zp[gi])::"memory");
  };
  auto wait_only = [&](auto n) { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(decltype(n)::value) : "memory"); };

  // Everything from here to the end of the main loop exists once per number of row tiles that are multiplied (WMV):
  // all WM of them, or - block at most half full - the lower WM/2 only.  The choice is made once per
  // workgroup, outside the scheduled loop; guarding single row tiles inside it would split the loop body into basic
  // blocks and lose the interleaving of LDS reads, conversions and MFMAs (measured: 20 % slower, not faster).
  auto run = [&](auto wmv_c) {
    constexpr int WMV = decltype(wmv_c)::value;
    // Fragments this wavefront stages per x stage.  A 256-slot expert block of which at most the lower eight row tiles
    // hold slots stages those only (two fragments per wavefront instead of four); the reads below never reach further.
    constexpr int APV = (GROUPED && WM == 16 && WMV <= 8) ? 2 : AP;
    uint32_t a_voff[APV / 2];
#pragma unroll
    for (int j = 0; j < APV / 2; ++j) {
      const uint32_t rb = wave * (APV / 2) + j;
      uint32_t row = rb * 16 + (lane >> 2);
      if (GROUPED) {
        uint32_t sid = static_cast<uint32_t>(p.sorted_ids[m0 + row]);
        sid = sid < p.numel ? sid : p.numel - 1;  // pad slots read some valid row; their results are dropped
        row = sid / p.top_k;
      } else {
        row = (m0 + row < p.M) ? row : (p.M - 1 - m0);  // rows past M repeat the last row; their results are dropped
      }
      a_voff[j] = (row * p.K + 8 * ((lane & 3) ^ (lane >> 4))) * 2;
    }
    const uint32_t a_lds_wave = lds_base + wave * APV * 1024;
    // x stage `stage` -> LDS slot stage % NS, fragment pair `part` of this wavefront's APV / 2 pairs.  The instruction
    // offset of an LDS-targeted load is added to the LDS address as well as to the global one: the second fragment's
    // 64-byte global offset is taken back out of its LDS base.
    auto load_a_part = [&](uint32_t stage, auto pc) {
      constexpr int part = decltype(pc)::value;
      if constexpr (part >= APV / 2) return;
      const uint32_t st = stage < stages ? stage : stages - 1;
      const char* src = x_tile + static_cast<size_t>(st) * (BK * 2);
      const uint32_t d0 = __builtin_amdgcn_readfirstlane(a_lds_wave + (stage % NS) * STAGE_BYTES) + part * 2048;
      const uint32_t d1 = d0 + 1024 - 64;
      const uint32_t av = a_voff[part < APV / 2 ? part : 0];
      asm volatile(
          "s_nop 4\n\t"
          "s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %3\n\t"
          "s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %3 offset:64"
          :
          : "v"(av), "s"(d0), "s"(d1), "s"(src)
          : "memory", "m0");
    };
    auto load_a = [&](uint32_t stage) {
      static_assert(APV == 2 || APV == 4, "one or two fragment pairs per wavefront and stage");
      load_a_part(stage, std::integral_constant<int, 0>{});
      load_a_part(stage, std::integral_constant<int, 1>{});
    };
    // ---- compute pipeline, in steps of 32 k (two per stage).  A fragments are read DEPTH ahead of the MFMAs that use
    // them, across step and stage boundaries; the weight fragments of step g+1 are dequantized while step g multiplies.
    constexpr int DEPTH = 4;
    // the prefetch ring runs on through the steps: a step of WMV reads leaves it turned by WMV % DEPTH places, and the
    // twelve steps of one turn of the main loop by a whole number of turns
    static_assert((12 * WMV) % DEPTH == 0 && WMV >= DEPTH, "the main loop must turn the A prefetch ring a whole number of times");
    u32x4 abuf[DEPTH];
    typename T::frag bfrag[2][WN];  // weight fragments of the current step [g % 2] and the next one
    Dequant<T, HAS_ZP> dq[WN];

    auto frag_ptr = [&](uint32_t slot, int ks) { return lds + slot * STAGE_BYTES + ks * 1024 + a_rd; };
    // `wn`/`dn`: weight slot and dword (32-k block of its k-tile) the NEXT step uses
    auto step = [&](auto parity, auto turn, uint32_t slot, int ks, WSlot (&wn)[WN], int dn, auto&& issue) {
      constexpr int P = decltype(parity)::value;
      constexpr int TURN = decltype(turn)::value;  // where the prefetch ring stands when this step starts
      typename T::frag(&bcur)[WN] = bfrag[P];
      typename T::frag(&bnext)[WN] = bfrag[P ^ 1];
      const char* cur = frag_ptr(slot, ks);
      const char* nxt = ks == 0 ? frag_ptr(slot, 1) : frag_ptr((slot + 1) % NS, 0);
      if (dn % (4 / GPT) == 0) {  // the next step opens a new quantization group
  #pragma unroll
        for (int t = 0; t < WN; ++t) dq[t].set(wn[t].sc[dn / (4 / GPT)], wn[t].zp[dn / (4 / GPT)]);
      }
  #pragma unroll
      for (int i = 0; i < WMV; ++i) {
        const u32x4 a = abuf[(i + TURN) % DEPTH];
        const int ni = i + DEPTH;
        abuf[(i + TURN) % DEPTH] = ni < WMV ? *reinterpret_cast<const u32x4*>(cur + ni * 2048)
                                   : *reinterpret_cast<const u32x4*>(nxt + (ni - WMV) * 2048);
  #pragma unroll
        for (int t = 0; t < WN; ++t) acc[t][i] = T::mfma(bcur[t], as_frag<T>(a), acc[t][i]);
        if (i == 1) bnext[0] = dq[0](wn[0].wq[dn]);
        if (i == WMV / 2 + 1) bnext[1] = dq[1](wn[1].wq[dn]);
        issue(std::integral_constant<int, 0>{}, i);
        __builtin_amdgcn_sched_barrier(0x6);  // VALU / SALU may move; LDS reads and MFMAs keep this order
      }
    };
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;

    // ---- schedule.  One synchronisation point per stage, in its middle ("sync c" sits between the two steps of
    // stage c): wait for x stage c+1, barrier.  x stage c+3 is issued during the second step of stage c - its LDS slot is
    // the one stage c-1 used, and every wavefront is past that -, the weights of k-tile (c+3)/2 during the first step of
    // the odd stages c: issued in stage 2kt-3, they are waited for at sync 2kt-2 and first dequantized during the last
    // step of k-tile kt-1.  Issue order around sync c: ... x(c+1) [w((c+2)/2), c even] x(c+2) [w((c+3)/2), c odd] | sync c:
    // after x stage c+1 (and, c even, the weights behind it) come APV loads when c is even, APV + 2*WL when c is odd.
    using WaitEven = std::integral_constant<int, APV>;
    using WaitOdd = std::integral_constant<int, APV + WN * WL>;
    using WaitFirst = std::integral_constant<int, 2 * APV + WN * WL>;
    load_w(ring[0], 0);
    load_a(0);
    load_w(ring[1], 1);
    load_a(1);
    load_a(2);
    wait_tie(WaitFirst{}, ring[0]);  // x stage 0 and k-tile 0 are in
    __builtin_amdgcn_s_barrier();
  #pragma unroll
    for (int t = 0; t < WN; ++t) {
      dq[t].set(ring[0][t].sc[0], ring[0][t].zp[0]);
      bfrag[0][t] = dq[t](ring[0][t].wq[0]);
    }
  #pragma unroll
    for (int j = 0; j < DEPTH; ++j) abuf[j] = *reinterpret_cast<const u32x4*>(frag_ptr(0, 0) + j * 2048);

    // stage base + u of the six stages (three k-tiles) one turn of the main loop covers
    auto stage = [&](auto uc, uint32_t base) {
      constexpr int u = decltype(uc)::value;
      using Turn0 = std::integral_constant<int, (2 * u * WMV) % DEPTH>;
      using Turn1 = std::integral_constant<int, ((2 * u + 1) * WMV) % DEPTH>;
      const uint32_t s = base + u;
      const uint32_t slot = s % NS;
      auto none = [](auto, int) {};
      // The loads are spread over the row tiles of the steps (one group per row tile) instead of issued in one run
      // behind the barrier, where all eight wavefronts queue at the memory pipeline at once: the weights of k-tile
      // s/2+2 during the first step of the odd stages (registers: no barrier to wait for), x stage s+3 during the
      // second step of every stage (its LDS slot is free once every wavefront is past the barrier).
      auto spread_w = [&](auto, int i) {
        if (i == 0) load_w_part(ring[(u / 2 + 2) % 3], s / 2 + 2, std::integral_constant<int, 0>{});
        if (i == 2) load_w_part(ring[(u / 2 + 2) % 3], s / 2 + 2, std::integral_constant<int, 1>{});
      };
      auto spread_a = [&](auto, int i) {
        if (i == 0) load_a_part(s + 3, std::integral_constant<int, 0>{});
        if (i == 2) load_a_part(s + 3, std::integral_constant<int, 1>{});
      };
      // first step of the stage: k block 2*(u%2) of k-tile u/2; the next step uses block 2*(u%2)+1 of the same tile
      if constexpr (u % 2 == 0) {
        if (s < stages) step(Even{}, Turn0{}, slot, 0, ring[(u / 2) % 3], 2 * (u % 2) + 1, none);
      } else {
        if (s < stages) {
          step(Even{}, Turn0{}, slot, 0, ring[(u / 2) % 3], 2 * (u % 2) + 1, spread_w);
        } else {
          spread_w(0, 0);
          spread_w(0, 2);
        }
      }
      // sync s
      if constexpr (u % 2 == 0) {
        wait_tie(WaitEven{}, ring[(u / 2 + 1) % 3]);  // k-tile s/2+1, issued during stage s-1
      } else {
        wait_only(WaitOdd{});
      }
      __builtin_amdgcn_s_barrier();
      // second step: the next step is block 2 of this k-tile (u even) or block 0 of the next k-tile (u odd)
      if (s < stages) {
        if constexpr (u % 2 == 0)
          step(Odd{}, Turn1{}, slot, 1, ring[(u / 2) % 3], 2, spread_a);
        else
          step(Odd{}, Turn1{}, slot, 1, ring[(u / 2 + 1) % 3], 0, spread_a);
      } else {
        spread_a(0, 0);
        spread_a(0, 2);
      }
    };
    for (uint32_t base = 0; base < stages; base += 6) {
      stage(std::integral_constant<int, 0>{}, base);
      stage(std::integral_constant<int, 1>{}, base);
      stage(std::integral_constant<int, 2>{}, base);
      stage(std::integral_constant<int, 3>{}, base);
      stage(std::integral_constant<int, 4>{}, base);
      stage(std::integral_constant<int, 5>{}, base);
    }
  };
  if (GROUPED) {
    // expert blocks: an instance of the main loop for every number of row tiles that hold slots, from four (the depth
    // of the fragment prefetch) to all of them.  What a padded row tile costs is not so much time in the loop as power
    // - its MFMAs multiply real rows -, and the clock: at 128 slots per expert on average, instances over 9 and 10
    // row tiles next to those over 8 and 12 took a tenth off the whole call.
    for_tile_count<4, WM>(live_tiles, run);
  } else if (live_tiles <= WM / 2) {
    run(std::integral_constant<int, WM / 2>{});
  } else {
    run(std::integral_constant<int, WM>{});
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // drain the clamped prefetches before the LDS is released

  // ---- store: lane holds row m = l%16 of the 16x16 tile and columns 4*(l/16) .. +3
  // Grouped form: the slot ids of all row tiles, then their routing weights, are fetched before the first store.  Read
  // inside the loop they would each wait for the stores in front of them (the compiler cannot know that the output
  // does not overlap the index arrays), one memory round trip after the other: 16 row tiles cost 15 us per
  // workgroup that way, a fifth of the whole launch at K = 2048.
  uint32_t sids[WM];
  float rws[WM];
  if (GROUPED) {
#pragma unroll
    for (int i = 0; i < WM; ++i) sids[i] = static_cast<uint32_t>(p.sorted_ids[m0 + i * 16 + lrow]);
#pragma unroll
    for (int i = 0; i < WM; ++i) rws[i] = (sids[i] < p.numel && p.topk_w) ? p.topk_w[sids[i]] : 1.0f;
  }
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    uint32_t row = m0 + i * 16 + lrow;
    bool live;
    float rw = 1.0f;
    if (GROUPED) {
      live = sids[i] < p.numel;
      row = sids[i];
      rw = rws[i];
    } else {
      live = row < p.M;
    }
    if (GROUPED && paired) {
      // T(silu(T(gate)) * T(up)): both sums rounded to T as the plain GEMM would store them, so that the result has the
      // bits of the two-launch form
      if (live && nt0 < p.pair_tiles) {
        u32x2 o;
        uint16_t h[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float gv = T::to_float(T::from_float(acc[0][i][j])), uv = T::to_float(T::from_float(acc[1][i][j]));
          h[j] = T::from_float(silu_mul_f32(gv, uv));
        }
        o.x = pack2(h[0], h[1]);
        o.y = pack2(h[2], h[3]);
        const size_t col = static_cast<size_t>(nt0) * 16 + 4 * lq;
        *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(p.y) + static_cast<size_t>(row) * (p.N / 2) + col) = o;
      }
    } else if (live) {
#pragma unroll
      for (int t = 0; t < WN; ++t) {
        if (nt0 + t < n_tiles) {
          const size_t col = static_cast<size_t>(nt0 + t) * 16 + 4 * lq;
          if (!GROUPED && direct && p.y32) {
            *reinterpret_cast<f32x4*>(p.y32 + static_cast<size_t>(row) * p.N + col) = acc[t][i];
          } else if (GROUPED || direct) {
            f32x4 v = acc[t][i];
            if (GROUPED) v *= rw;
            u32x2 o;
            o.x = pack2(T::from_float(v[0]), T::from_float(v[1]));
            o.y = pack2(T::from_float(v[2]), T::from_float(v[3]));
            *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(p.y) + static_cast<size_t>(row) * p.N + col) = o;
          } else {
            float* dst = p.partial + ((static_cast<size_t>(slot) * p.splits + part) * BM + (row - m0)) * BN + (col - n0);
            *reinterpret_cast<f32x4*>(dst) = acc[t][i];
          }
        }
      }
    }
  }
}

}  // namespace ksq
