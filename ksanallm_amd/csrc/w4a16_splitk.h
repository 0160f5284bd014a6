// Decode-regime W4A16 kernel (small M, HBM-bound): split-K across the wavefronts of a workgroup.
//
// A workgroup owns NT tiles of 16 output columns and MT tiles of 16 rows of x.  Wavefront w walks the 128-wide
// k-tiles w, w+WAVES, ... ; per k-tile each lane loads 16 bytes of packed codes per column tile (one coalesced 1 KiB
// wavefront load), turns every dword into an MFMA operand holding magic+code with four and-or instructions, and
// feeds v_mfma_f32_16x16x32 with the weights as the row operand and x as the column operand.  The group's zero point
// and scale are applied to the fp32 partial afterwards:
//     acc += s * (sum_k x*(magic+code) - (magic+zp) * sum_k x)
// where sum_k x comes from one more MFMA against an all-ones operand, so nothing but and-or work runs on the VALU
// per weight.  The wavefronts' partials meet in LDS and are summed in wavefront order (deterministic).
//
// The same kernel serves the MoE grouped GEMM: rows come from sorted slot ids, the expert of the block selects the
// weight slab, and the routed weight is applied on the way out.
#pragma once

#include "ksq_common.h"

namespace ksq {

struct SplitKParams {
  void* y;
  const void* x;
  const u32x4* w;
  const uint16_t* scales;
  const uint8_t* zeros;
  uint32_t M, N, K;
  // grouped (MoE) mode
  const int32_t* sorted_ids;
  const int32_t* expert_ids;
  const int32_t* num_post_pad;
  const float* topk_w;
  uint32_t numel, top_k;
};

template <typename T, int MT, int NT, int WAVES, int GROUP, bool HAS_ZP, bool GROUPED>
__global__ void __launch_bounds__(WAVES * 64) w4a16_splitk_kernel(SplitKParams p) {
  constexpr int GPT = 128 / GROUP;  // groups per k-tile
  constexpr int SPG = GROUP / 32;   // MFMA k-steps per group
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int lrow = lane & 15;
  const int lq = lane >> 4;
  const uint32_t KT = p.K / 128;
  const uint32_t G = p.K / GROUP;
  const uint32_t nt0 = blockIdx.x * NT;

  __shared__ f32x4 red[WAVES][NT * MT][64];

  // ---- which rows of x this lane feeds, and where they go
  uint32_t xrow[MT];
  bool ok[MT];
  size_t tile_base = 0;  // first weight tile of the expert, in tiles
  size_t sz_base = 0;    // first scale / zero element of the expert
  if (GROUPED) {
    const uint32_t pos0 = blockIdx.y * (16 * MT);
    if (pos0 >= static_cast<uint32_t>(p.num_post_pad[0])) return;
    const uint32_t e = static_cast<uint32_t>(p.expert_ids[blockIdx.y]);
    tile_base = static_cast<size_t>(e) * (p.N / 16) * KT;
    sz_base = static_cast<size_t>(e) * G * p.N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      uint32_t sid = static_cast<uint32_t>(p.sorted_ids[pos0 + mt * 16 + lrow]);
      ok[mt] = sid < p.numel;
      xrow[mt] = sid / p.top_k;
    }
  } else {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      xrow[mt] = blockIdx.y * (16 * MT) + mt * 16 + lrow;
      ok[mt] = xrow[mt] < p.M;
    }
  }

  const u32x4* wbase[NT];
  const uint16_t* sbase[NT];
  const uint8_t* zbase[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    wbase[t] = p.w + (tile_base + static_cast<size_t>(nt0 + t) * KT) * 64 + lane;
    sbase[t] = p.scales + sz_base + static_cast<size_t>(nt0 + t) * G * 16 + 4 * lq;
    zbase[t] = HAS_ZP ? p.zeros + sz_base + static_cast<size_t>(nt0 + t) * G * 16 + 4 * lq : nullptr;
  }
  const uint16_t* xbase[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    xbase[mt] = static_cast<const uint16_t*>(p.x) + static_cast<size_t>(xrow[mt]) * p.K + lq * 8;

  f32x4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct Stage {
    u32x4 wq[NT];
    u32x4 xf[MT][4];
    u32x2 sc[NT][GPT];
    uint32_t zp[NT][GPT];
  };

  auto load_stage = [&](Stage& s, uint32_t kt) {
#pragma unroll
    for (int t = 0; t < NT; ++t) s.wq[t] = __builtin_nontemporal_load(wbase[t] + static_cast<size_t>(kt) * 64);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int d = 0; d < 4; ++d)
        s.xf[mt][d] = ok[mt] ? *reinterpret_cast<const u32x4*>(xbase[mt] + kt * 128 + d * 32) : u32x4{0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi) {
        s.sc[t][gi] = *reinterpret_cast<const u32x2*>(sbase[t] + (static_cast<size_t>(kt) * GPT + gi) * 16);
        if (HAS_ZP) s.zp[t][gi] = *reinterpret_cast<const uint32_t*>(zbase[t] + (static_cast<size_t>(kt) * GPT + gi) * 16);
      }
  };

  const typename T::frag ones = as_frag<T>(u32x4{T::kOne2, T::kOne2, T::kOne2, T::kOne2});

  auto compute_stage = [&](const Stage& s) {
#pragma unroll
    for (int gi = 0; gi < GPT; ++gi) {
      float sx[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        f32x4 r{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = gi * SPG; d < (gi + 1) * SPG; ++d) r = T::mfma(ones, as_frag<T>(s.xf[mt][d]), r);
        sx[mt] = r.x;
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        float sc[4], cz[4];
        sc[0] = T::to_float(static_cast<uint16_t>(s.sc[t][gi].x & 0xffffu));
        sc[1] = T::to_float(static_cast<uint16_t>(s.sc[t][gi].x >> 16));
        sc[2] = T::to_float(static_cast<uint16_t>(s.sc[t][gi].y & 0xffffu));
        sc[3] = T::to_float(static_cast<uint16_t>(s.sc[t][gi].y >> 16));
#pragma unroll
        for (int i = 0; i < 4; ++i)
          cz[i] = HAS_ZP ? T::kMagic + static_cast<float>((s.zp[t][gi] >> (8 * i)) & 0xffu) : T::kMagic + 8.0f;
        typename T::frag wf[SPG];
#pragma unroll
        for (int d = 0; d < SPG; ++d) wf[d] = dequant_magic<T>(s.wq[t][gi * SPG + d]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          f32x4 r{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int d = 0; d < SPG; ++d) r = T::mfma(wf[d], as_frag<T>(s.xf[mt][gi * SPG + d]), r);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[t][mt][i] += sc[i] * (r[i] - cz[i] * sx[mt]);
        }
      }
    }
  };

  // ---- main loop, one stage of loads in flight ahead of the math
  uint32_t kt = wave;
  if (kt < KT) {
    Stage cur;
    load_stage(cur, kt);
    for (;;) {
      uint32_t nk = kt + WAVES;
      if (nk < KT) {
        Stage nxt;
        load_stage(nxt, nk);
        compute_stage(cur);
        cur = nxt;
        kt = nk;
      } else {
        compute_stage(cur);
        break;
      }
    }
  }

  // ---- cross-wavefront reduction in wavefront order
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[wave][t * MT + mt][lane] = acc[t][mt];
  __syncthreads();

  for (int idx = threadIdx.x; idx < NT * MT * 64; idx += WAVES * 64) {
    const int l = idx & 63;
    const int tm = idx >> 6;
    const int t = tm / MT, mt = tm % MT;
    f32x4 v = red[0][tm][l];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) v += red[w][tm][l];
    uint32_t orow;
    bool valid;
    float rw = 1.0f;
    if (GROUPED) {
      uint32_t sid = static_cast<uint32_t>(p.sorted_ids[blockIdx.y * (16 * MT) + mt * 16 + (l & 15)]);
      valid = sid < p.numel;
      orow = sid;
      if (valid && p.topk_w) rw = p.topk_w[sid];
    } else {
      orow = blockIdx.y * (16 * MT) + mt * 16 + (l & 15);
      valid = orow < p.M;
    }
    if (valid) {
      u32x2 o;
      o.x = pack2(T::from_float(v[0] * rw), T::from_float(v[1] * rw));
      o.y = pack2(T::from_float(v[2] * rw), T::from_float(v[3] * rw));
      uint16_t* yp = static_cast<uint16_t*>(p.y) + static_cast<size_t>(orow) * p.N + (nt0 + t) * 16 + 4 * (l >> 4);
      *reinterpret_cast<u32x2*>(yp) = o;
    }
  }
}

}  // namespace ksq
