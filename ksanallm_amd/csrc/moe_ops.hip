// MoE helpers around the grouped GEMM: expert-offset / permutation build, silu*mul, top-k sum.
#include "ksq_common.h"

namespace ksq {
namespace {

constexpr int kAlignThreads = 1024;

// Stable counting sort by expert in one workgroup.
//   chunk c (one thread) owns ids [c*per, (c+1)*per); cnt[c+1][e] = #ids == e in chunk c  (global scratch)
//   column scan over chunks turns cnt[c][e] into "ids == e before chunk c";  padded totals are scanned over experts
//   in LDS; every chunk then places its ids in order, so positions inside an expert ascend with the flat index.
__global__ void __launch_bounds__(kAlignThreads) moe_align_kernel(const int32_t* __restrict__ ids, uint32_t numel,
                                                                  uint32_t E, uint32_t block_m, uint32_t capacity,
                                                                  int32_t* __restrict__ sorted, int32_t* __restrict__ expert_ids,
                                                                  int32_t* __restrict__ num_post_pad,
                                                                  int32_t* __restrict__ cnt, uint32_t chunks,
                                                                  uint32_t per) {
  extern __shared__ int32_t lds[];  // [2][E_pad + 1] ping-pong scan buffers
  const uint32_t tid = threadIdx.x;
  const uint32_t EP = E + 1;
  int32_t* scan_a = lds;
  int32_t* scan_b = lds + EP;

  // fill: every slot starts as padding
  for (uint32_t i = tid; i < capacity; i += kAlignThreads) sorted[i] = static_cast<int32_t>(numel);
  // clear counters
  for (uint32_t i = tid; i < (chunks + 1) * E; i += kAlignThreads) cnt[i] = 0;
  __syncthreads();

  const uint32_t begin = tid * per;
  const uint32_t end = (begin + per < numel) ? begin + per : numel;
  if (tid < chunks) {
    for (uint32_t i = begin; i < end; ++i) {
      uint32_t e = static_cast<uint32_t>(ids[i]);
      if (e < E) cnt[(tid + 1) * E + e] += 1;
    }
  }
  __syncthreads();

  // per expert: running sum over chunks
  for (uint32_t e = tid; e < E; e += kAlignThreads) {
    int32_t run = 0;
    for (uint32_t c = 1; c <= chunks; ++c) {
      run += cnt[c * E + e];
      cnt[c * E + e] = run;
    }
    // cnt[chunks][e] == total of expert e ; padded size goes into the scan buffer (shifted by one: exclusive scan)
    scan_a[e + 1] = (run + static_cast<int32_t>(block_m) - 1) / static_cast<int32_t>(block_m) * static_cast<int32_t>(block_m);
  }
  if (tid == 0) scan_a[0] = 0;
  __syncthreads();

  // inclusive Hillis-Steele scan over EP entries -> scan[e] = first slot of expert e, scan[E] = padded total
  int32_t* src = scan_a;
  int32_t* dst = scan_b;
  for (uint32_t off = 1; off < EP; off <<= 1) {
    for (uint32_t i = tid; i < EP; i += kAlignThreads) dst[i] = src[i] + (i >= off ? src[i - off] : 0);
    __syncthreads();
    int32_t* t = src;
    src = dst;
    dst = t;
  }
  const int32_t* first = src;

  if (tid == 0) num_post_pad[0] = first[E];
  for (uint32_t e = tid; e < E; e += kAlignThreads)
    for (int32_t s = first[e]; s < first[e + 1]; s += static_cast<int32_t>(block_m)) expert_ids[s / static_cast<int32_t>(block_m)] = static_cast<int32_t>(e);

  if (tid < chunks) {
    for (uint32_t i = begin; i < end; ++i) {
      uint32_t e = static_cast<uint32_t>(ids[i]);
      if (e < E) {
        int32_t r = cnt[tid * E + e];
        cnt[tid * E + e] = r + 1;
        sorted[first[e] + r] = static_cast<int32_t>(i);
      }
    }
  }
}

// ---- the same sort for up to 1024 ids (decode batches), one id per thread, everything in LDS: no counter ever makes
// a round trip through global memory, which is what the launch above spends most of its microseconds on.
//   r        = lower lanes of the wavefront with the same id (64 readlanes)
//   wcnt[w][e] = ids == e in wavefront w, then, scanned over w, ids == e in the wavefronts before w
//   position = first[e] + wcnt[w][e] + r : ascending with the flat index inside an expert, as above
__global__ void __launch_bounds__(1024) moe_align_small_kernel(const int32_t* __restrict__ ids, uint32_t numel, uint32_t E,
                                                               uint32_t block_m, uint32_t capacity,
                                                               int32_t* __restrict__ sorted, int32_t* __restrict__ expert_ids,
                                                               int32_t* __restrict__ num_post_pad) {
  extern __shared__ int32_t lds[];  // wcnt[W][E], then [2][E + 1] ping-pong scan buffers
  const uint32_t tid = threadIdx.x, threads = blockDim.x;
  const uint32_t lane = tid & 63, wave = tid >> 6;
  const uint32_t W = (numel + 63) / 64;
  const uint32_t EP = E + 1;
  int32_t* wcnt = lds;
  int32_t* scan_a = lds + W * E;
  int32_t* scan_b = scan_a + EP;

  for (uint32_t i = tid; i < capacity; i += threads) sorted[i] = static_cast<int32_t>(numel);  // every slot starts as padding
  for (uint32_t i = tid; i < W * E; i += threads) wcnt[i] = 0;

  const uint32_t id = tid < numel ? static_cast<uint32_t>(ids[tid]) : 0xffffffffu;
  const bool valid = id < E;
  uint32_t r = 0;
  bool last = true;
#pragma unroll
  for (int l = 0; l < 64; ++l) {
    const uint32_t v = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(id), l));
    const bool same = v == id;
    r += (same && static_cast<uint32_t>(l) < lane) ? 1u : 0u;
    last = last && !(same && static_cast<uint32_t>(l) > lane);
  }
  __syncthreads();
  if (valid && last) wcnt[wave * E + id] = static_cast<int32_t>(r + 1);
  __syncthreads();

  for (uint32_t e = tid; e < E; e += threads) {
    int32_t run = 0;
    for (uint32_t w = 0; w < W; ++w) {
      const int32_t c = wcnt[w * E + e];
      wcnt[w * E + e] = run;
      run += c;
    }
    scan_a[e + 1] = (run + static_cast<int32_t>(block_m) - 1) / static_cast<int32_t>(block_m) * static_cast<int32_t>(block_m);
  }
  if (tid == 0) scan_a[0] = 0;
  __syncthreads();

  int32_t* src = scan_a;
  int32_t* dst = scan_b;
  for (uint32_t off = 1; off < EP; off <<= 1) {
    for (uint32_t i = tid; i < EP; i += threads) dst[i] = src[i] + (i >= off ? src[i - off] : 0);
    __syncthreads();
    int32_t* t = src;
    src = dst;
    dst = t;
  }
  const int32_t* first = src;

  if (tid == 0) num_post_pad[0] = first[E];
  for (uint32_t e = tid; e < E; e += threads)
    for (int32_t p = first[e]; p < first[e + 1]; p += static_cast<int32_t>(block_m)) expert_ids[p / static_cast<int32_t>(block_m)] = static_cast<int32_t>(e);
  if (valid) sorted[first[id] + wcnt[wave * E + id] + static_cast<int32_t>(r)] = static_cast<int32_t>(tid);
}

// ---- the same sort for many ids: two launches over `chunks` workgroups ---------------------------------------------
constexpr int kChunkThreads = 256;
constexpr uint32_t kMaxChunks = 128;

// Launch 1: workgroup c counts its chunk's ids per expert into cnt[c][e]; all workgroups together fill `sorted` with
// the padding value.
__global__ void __launch_bounds__(kChunkThreads) moe_align_count_kernel(const int32_t* __restrict__ ids, uint32_t numel,
                                                                        uint32_t E, uint32_t capacity,
                                                                        int32_t* __restrict__ sorted,
                                                                        int32_t* __restrict__ cnt, uint32_t per) {
  extern __shared__ int32_t lds[];  // [E]
  const uint32_t tid = threadIdx.x;
  for (uint32_t e = tid; e < E; e += kChunkThreads) lds[e] = 0;
  for (uint32_t i = blockIdx.x * kChunkThreads + tid; i < capacity; i += gridDim.x * kChunkThreads)
    sorted[i] = static_cast<int32_t>(numel);
  __syncthreads();
  const uint32_t begin = blockIdx.x * per;
  const uint32_t end = (begin + per < numel) ? begin + per : numel;
  for (uint32_t i = begin + tid; i < end; i += kChunkThreads) {
    uint32_t e = static_cast<uint32_t>(ids[i]);
    if (e < E) atomicAdd(&lds[e], 1);
  }
  __syncthreads();
  for (uint32_t e = tid; e < E; e += kChunkThreads) cnt[blockIdx.x * E + e] = lds[e];
}

// Launch 2: every workgroup sums the count table (ids of each expert before its chunk, and in total), scans the padded
// totals over experts, and places its chunk's ids in rounds of 256: inside a round an id's rank is the number of equal
// ids at lower positions, so the order inside an expert ascends with the flat index.  Workgroup 0 also writes
// expert_ids and num_post_pad.
__global__ void __launch_bounds__(kChunkThreads) moe_align_place_kernel(const int32_t* __restrict__ ids, uint32_t numel,
                                                                        uint32_t E, uint32_t block_m,
                                                                        int32_t* __restrict__ sorted,
                                                                        int32_t* __restrict__ expert_ids,
                                                                        int32_t* __restrict__ num_post_pad,
                                                                        const int32_t* __restrict__ cnt, uint32_t chunks,
                                                                        uint32_t per) {
  extern __shared__ int32_t lds[];  // scan_a[E+1] scan_b[E+1] next[E] round[256]
  const uint32_t tid = threadIdx.x;
  const uint32_t EP = E + 1;
  int32_t* scan_a = lds;
  int32_t* scan_b = lds + EP;
  int32_t* next = lds + 2 * EP;
  int32_t* round = next + E;
  const uint32_t c = blockIdx.x;
  const int32_t bm = static_cast<int32_t>(block_m);

  for (uint32_t e = tid; e < E; e += kChunkThreads) {
    int32_t before = 0, total = 0;
#pragma unroll 8
    for (uint32_t c2 = 0; c2 < chunks; ++c2) {
      int32_t v = cnt[c2 * E + e];
      total += v;
      before += (c2 < c) ? v : 0;
    }
    next[e] = before;
    scan_a[e + 1] = (total + bm - 1) / bm * bm;
  }
  if (tid == 0) scan_a[0] = 0;
  __syncthreads();
  int32_t* src = scan_a;
  int32_t* dst = scan_b;
  for (uint32_t off = 1; off < EP; off <<= 1) {
    for (uint32_t i = tid; i < EP; i += kChunkThreads) dst[i] = src[i] + (i >= off ? src[i - off] : 0);
    __syncthreads();
    int32_t* t = src;
    src = dst;
    dst = t;
  }
  const int32_t* first = src;
  if (c == 0) {
    if (tid == 0) num_post_pad[0] = first[E];
    for (uint32_t e = tid; e < E; e += kChunkThreads)
      for (int32_t s = first[e]; s < first[e + 1]; s += bm) expert_ids[s / bm] = static_cast<int32_t>(e);
  }
  for (uint32_t e = tid; e < E; e += kChunkThreads) next[e] += first[e];
  __syncthreads();

  const uint32_t begin = c * per;
  const uint32_t end = (begin + per < numel) ? begin + per : numel;
  for (uint32_t r0 = begin; r0 < end; r0 += kChunkThreads) {
    const uint32_t i = r0 + tid;
    uint32_t e = (i < end) ? static_cast<uint32_t>(ids[i]) : 0xffffffffu;
    if (e >= E) e = 0xffffffffu;
    round[tid] = static_cast<int32_t>(e);
    __syncthreads();
    int32_t pos = 0;
    bool last = true;
    if (e != 0xffffffffu) {
      int32_t rank = 0;
      for (uint32_t j = 0; j < kChunkThreads; ++j) {
        const bool same = static_cast<uint32_t>(round[j]) == e;
        rank += (same && j < tid) ? 1 : 0;
        last = last && !(same && j > tid);
      }
      pos = next[e] + rank;
      sorted[pos] = static_cast<int32_t>(i);
    }
    __syncthreads();
    if (e != 0xffffffffu && last) next[e] = pos + 1;
    __syncthreads();
  }
}

void chunk_geometry(size_t numel, uint32_t* chunks, uint32_t* per) {
  size_t c = div_up(numel, kChunkThreads);
  if (c > kMaxChunks) c = kMaxChunks;
  const size_t p = div_up(div_up(numel, c), kChunkThreads) * kChunkThreads;
  *per = static_cast<uint32_t>(p);
  *chunks = static_cast<uint32_t>(div_up(numel, p));
}

// ids from which the two-launch sort is used
constexpr size_t kParallelAlignFrom = 2048;

// 8 elements per thread.  A workgroup covers 2^log2p column pieces of 256 >> log2p rows; the row comes from
// blockIdx.y/z, the column piece from blockIdx.x, so that no index is divided (a 64-bit division is some fifty
// instructions on this ISA, more than the rest of the kernel).
template <typename T>
__global__ void __launch_bounds__(256) silu_mul_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ out,
                                                       size_t rows, uint32_t inter, uint32_t log2p) {
  const uint32_t piece = (blockIdx.x << log2p) + (threadIdx.x & ((1u << log2p) - 1));
  const size_t r = (static_cast<size_t>(blockIdx.z) * gridDim.y + blockIdx.y) * (256u >> log2p) + (threadIdx.x >> log2p);
  if (piece >= inter / 8 || r >= rows) return;
  const uint32_t c = piece * 8;
  const uint16_t* a = x + r * 2 * inter + c;
  u32x4 ra = *reinterpret_cast<const u32x4*>(a);
  u32x4 rb = *reinterpret_cast<const u32x4*>(a + inter);
  u32x4 o;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float a0 = T::to_float(static_cast<uint16_t>(ra[j] & 0xffffu)), a1 = T::to_float(static_cast<uint16_t>(ra[j] >> 16));
    float b0 = T::to_float(static_cast<uint16_t>(rb[j] & 0xffffu)), b1 = T::to_float(static_cast<uint16_t>(rb[j] >> 16));
    float y0 = silu_mul_f32(a0, b0);
    float y1 = silu_mul_f32(a1, b1);
    o[j] = pack2(T::from_float(y0), T::from_float(y1));
  }
  *reinterpret_cast<u32x4*>(out + r * inter + c) = o;
}

// sum over top-k in T precision, ascending j (each partial sum is rounded to T like the reference's `scalar_t x`)
template <typename T>
__global__ void __launch_bounds__(256) moe_sum_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                      size_t tokens, uint32_t topk, uint32_t d) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t per_row = d / 8;
  if (i >= tokens * per_row) return;
  const size_t t = i / per_row;
  const uint32_t c = static_cast<uint32_t>(i % per_row) * 8;
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  // four rows are fetched before the first of them is added: the sums form a chain (each is rounded to T), the loads
  // need not wait for it
  const uint16_t* src = in + t * topk * d + c;
  for (uint32_t s0 = 0; s0 < topk; s0 += 4) {
    u32x4 r[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t sr = s0 + u < topk ? s0 + u : topk - 1;  // rows past the end repeat the last one and are not added
      r[u] = *reinterpret_cast<const u32x4*>(src + static_cast<size_t>(sr) * d);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (s0 + u < topk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[2 * j] = T::to_float(T::from_float(acc[2 * j] + T::to_float(static_cast<uint16_t>(r[u][j] & 0xffffu))));
          acc[2 * j + 1] = T::to_float(T::from_float(acc[2 * j + 1] + T::to_float(static_cast<uint16_t>(r[u][j] >> 16))));
        }
      }
    }
  }
  u32x4 o;
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = pack2(T::from_float(acc[2 * j]), T::from_float(acc[2 * j + 1]));
  *reinterpret_cast<u32x4*>(out + t * d + c) = o;
}

// ---- reductions over a whole wavefront, every lane active, result in every lane.  Four DPP row operations leave each
// row of 16 lanes with its result, four readlanes combine the rows: a few dozen cycles, where a butterfly of LDS-crossbar
// permutes (what __shfl_xor compiles to) costs several hundred - and the routers are nothing but chains of these.
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(float, dpp_u32<CTRL>(__builtin_bit_cast(uint32_t, v)));
}
__device__ __forceinline__ uint32_t lane_u32(uint32_t v, int l) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), l));
}
__device__ __forceinline__ float lane_f32(float v, int l) {
  return __builtin_bit_cast(float, lane_u32(__builtin_bit_cast(uint32_t, v), l));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f32<kDppXor1>(v));
  v = fmaxf(v, dpp_f32<kDppXor2>(v));
  v = fmaxf(v, dpp_f32<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_f32<kDppMirror>(v));
  return fmaxf(fmaxf(lane_f32(v, 0), lane_f32(v, 16)), fmaxf(lane_f32(v, 32), lane_f32(v, 48)));
}
// the partners of every step hold equal partial sums, so all lanes of a row end with the same bits
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f32<kDppXor1>(v);
  v += dpp_f32<kDppXor2>(v);
  v += dpp_f32<kDppHalfMirror>(v);
  v += dpp_f32<kDppMirror>(v);
  return (lane_f32(v, 0) + lane_f32(v, 16)) + (lane_f32(v, 32) + lane_f32(v, 48));
}
// A lane's candidate: the largest key wins, among equal keys the lower id; id 0xffffffff = no candidate.  pay travels
// with the winner.
struct Pick {
  float key, pay;
  uint32_t id;
};
constexpr uint32_t kNoPick = 0xffffffffu;
__device__ __forceinline__ bool beats(const Pick& a, const Pick& b) {
  return a.id != kNoPick && (b.id == kNoPick || a.key > b.key || (a.key == b.key && a.id < b.id));
}
template <int CTRL>
__device__ __forceinline__ void pick_step(Pick& p) {
  const Pick o{dpp_f32<CTRL>(p.key), dpp_f32<CTRL>(p.pay), dpp_u32<CTRL>(p.id)};
  if (beats(o, p)) p = o;
}
__device__ __forceinline__ Pick wave_argmax(Pick p) {
  pick_step<kDppXor1>(p);
  pick_step<kDppXor2>(p);
  pick_step<kDppHalfMirror>(p);
  pick_step<kDppMirror>(p);
  Pick r{lane_f32(p.key, 0), lane_f32(p.pay, 0), lane_u32(p.id, 0)};
#pragma unroll
  for (int row = 16; row < 64; row += 16) {
    const Pick o{lane_f32(p.key, row), lane_f32(p.pay, row), lane_u32(p.id, row)};
    if (beats(o, r)) r = o;
  }
  return r;
}

// one wavefront per token: lane l holds experts l, l+64, ... (NV each: 4 serves up to 256 experts, 16 up to 1024; a lone
// wavefront is bound by its instruction count, and every scan below runs NV times)
template <typename LOAD, int NV>
__global__ void __launch_bounds__(256) topk_softmax_kernel(const void* __restrict__ gating, float* __restrict__ topk_w,
                                                           int32_t* __restrict__ topk_ids, uint32_t tokens,
                                                           uint32_t E, uint32_t top_k, int norm, float scaling) {
  const uint32_t token = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (token >= tokens) return;
  float v[NV];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const uint32_t e = j * 64 + lane;
    v[j] = e < E ? LOAD::get(gating, static_cast<size_t>(token) * E + e) : -INFINITY;
    mx = fmaxf(mx, v[j]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const uint32_t e = j * 64 + lane;
    v[j] = e < E ? expf(v[j] - mx) : -1.0f;  // -1 never wins the arg-max below
    sum += e < E ? v[j] : 0.f;
  }
  sum = wave_sum(sum);
  float picked_sum = 0.f;
  float my_w = 0.f;
  int my_id = 0;
  for (uint32_t r = 0; r < top_k; ++r) {
    float best = -2.0f;
    uint32_t best_e = 0xffffffffu;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const uint32_t e = j * 64 + lane;
      if (v[j] > best) {  // ascending e inside a lane: strict > keeps the lower id on ties
        best = v[j];
        best_e = e;
      }
    }
    {
      const Pick w = wave_argmax(Pick{best, 0.f, best_e});
      best = w.key;
      best_e = w.id;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (static_cast<uint32_t>(j * 64 + lane) == best_e) v[j] = -1.0f;
    const float prob = best / sum;
    picked_sum += prob;
    if (static_cast<uint32_t>(lane) == r) {
      my_w = prob;
      my_id = static_cast<int>(best_e);
    }
  }
  if (static_cast<uint32_t>(lane) < top_k) {
    const float w = norm ? my_w / picked_sum : my_w;
    topk_w[static_cast<size_t>(token) * top_k + lane] = w * scaling;
    topk_ids[static_cast<size_t>(token) * top_k + lane] = my_id;
  }
}

struct LoadF32 {
  static __device__ __forceinline__ float get(const void* p, size_t i) { return static_cast<const float*>(p)[i]; }
};
template <typename T>
struct Load16 {
  static __device__ __forceinline__ float get(const void* p, size_t i) { return T::to_float(static_cast<const uint16_t*>(p)[i]); }
};

// Grouped routing (DeepSeek-V2/V3): one wavefront per token, lane l holds experts l, l+64, ... (NV each, as above).
//   score   = softmax(gating) or sigmoid(gating), fp32
//   choose  = score + bias (bias given) or score
//   group g = experts [g*per_group, (g+1)*per_group): its rank value is the sum of its two largest choose values
//             (bias given) or its largest one; the topk_group best groups stay, all other experts are out
//   top_k rounds of wave arg-max over choose pick the experts (descending, the lower id wins ties); the routing
//   weight of a pick is its score (without bias), divided by the sum of the picks when renormalize, times scaling.
// Group rank values are built from the choose values staged in LDS (one row of E floats per wavefront).
template <typename LOAD, int NV>
__global__ void __launch_bounds__(256) grouped_topk_kernel(const void* __restrict__ gating, const float* __restrict__ bias,
                                                           float* __restrict__ topk_w, int32_t* __restrict__ topk_ids,
                                                           uint32_t tokens, uint32_t E, uint32_t top_k, uint32_t groups,
                                                           uint32_t topk_group, int sigmoid, int renorm, float scaling) {
  extern __shared__ float lds_choose[];  // [4][E]
  const uint32_t wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const uint32_t token_raw = blockIdx.x * 4 + wave;
  const bool active = token_raw < tokens;
  const uint32_t token = active ? token_raw : tokens - 1;  // idle wavefronts repeat the last token and store nothing
  const uint32_t per_group = E / groups;
  float* choose_row = lds_choose + wave * E;

  float score[NV], choose[NV];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const uint32_t e = j * 64 + lane;
    score[j] = e < E ? LOAD::get(gating, static_cast<size_t>(token) * E + e) : -INFINITY;
    mx = fmaxf(mx, score[j]);
  }
  if (sigmoid) {
#pragma unroll
    for (int j = 0; j < NV; ++j) score[j] = 1.0f / (1.0f + expf(-score[j]));
  } else {
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const uint32_t e = j * 64 + lane;
      score[j] = e < E ? expf(score[j] - mx) : 0.f;
      sum += score[j];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int j = 0; j < NV; ++j) score[j] = score[j] / sum;
  }
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const uint32_t e = j * 64 + lane;
    choose[j] = e < E ? score[j] + (bias ? bias[e] : 0.f) : -INFINITY;
    if (e < E) choose_row[e] = choose[j];
  }
  __syncthreads();

  // rank value of a group (groups <= 64): the two largest choose values of group `grp` are found by LPG adjacent lanes,
  // each scanning every LPG-th value of the group, and merged over those lanes (LPG is 8, 4, 2 or 1: the merges stay
  // inside aligned runs of LPG lanes, and a run of lanes past the last group only ever merges with itself)
  const uint32_t lpg = groups <= 8 ? 8u : (groups <= 16 ? 4u : (groups <= 32 ? 2u : 1u));
  const uint32_t grp = static_cast<uint32_t>(lane) / lpg, slice = static_cast<uint32_t>(lane) % lpg;
  float m1 = -INFINITY, m2 = -INFINITY;
  if (grp < groups) {
    const float* g = choose_row + grp * per_group;
    for (uint32_t i = slice; i < per_group; i += lpg) {
      const float c = g[i];
      if (c > m1) {
        m2 = m1;
        m1 = c;
      } else if (c > m2) {
        m2 = c;
      }
    }
  }
  auto merge_top2 = [&](float o1, float o2) {
    const float lo = fminf(m1, o1);
    m1 = fmaxf(m1, o1);
    m2 = fmaxf(lo, fmaxf(m2, o2));
  };
  if (lpg >= 2) merge_top2(dpp_f32<kDppXor1>(m1), dpp_f32<kDppXor1>(m2));
  if (lpg >= 4) merge_top2(dpp_f32<kDppXor2>(m1), dpp_f32<kDppXor2>(m2));
  if (lpg >= 8) merge_top2(dpp_f32<kDppHalfMirror>(m1), dpp_f32<kDppHalfMirror>(m2));
  const float rank = grp < groups ? (bias ? m1 + m2 : m1) : -INFINITY;
  uint64_t kept = 0;
  for (uint32_t r = 0; r < topk_group; ++r) {
    float best = rank;
    uint32_t best_g = (grp < groups && slice == 0) ? grp : 0xffffffffu;  // one lane per group carries its candidate
    if (grp < groups && ((kept >> grp) & 1)) best_g = 0xffffffffu;  // taken: never wins
    best_g = wave_argmax(Pick{best, 0.f, best_g}).id;
    if (best_g != 0xffffffffu) kept |= 1ull << best_g;
  }
  uint32_t taken = 0;  // bit j: expert j*64+lane is out (group not kept, past E, or already picked)
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const uint32_t e = j * 64 + lane;
    if (e >= E || !((kept >> (e / per_group)) & 1)) taken |= 1u << j;
  }

  float picked_sum = 0.f, my_w = 0.f;
  int my_id = 0;
  for (uint32_t r = 0; r < top_k; ++r) {
    float best = 0.f, best_s = 0.f;
    uint32_t best_e = 0xffffffffu;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      if (!((taken >> j) & 1) && (best_e == 0xffffffffu || choose[j] > best)) {  // ascending e: > keeps the lower id
        best = choose[j];
        best_s = score[j];
        best_e = j * 64 + lane;
      }
    }
    {
      const Pick w = wave_argmax(Pick{best, best_s, best_e});
      best_s = w.pay;
      best_e = w.id;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (static_cast<uint32_t>(j * 64 + lane) == best_e) taken |= 1u << j;
    picked_sum += best_s;
    if (static_cast<uint32_t>(lane) == r) {
      my_w = best_s;
      my_id = static_cast<int>(best_e);
    }
  }
  if (active && static_cast<uint32_t>(lane) < top_k) {
    const float w = renorm ? my_w / picked_sum : my_w;
    topk_w[static_cast<size_t>(token) * top_k + lane] = w * scaling;
    topk_ids[static_cast<size_t>(token) * top_k + lane] = my_id;
  }
}

void align_geometry(size_t numel, uint32_t* chunks, uint32_t* per) {
  size_t c = div_up(numel, 8);
  if (c < 1) c = 1;
  if (c > kAlignThreads) c = kAlignThreads;
  *chunks = static_cast<uint32_t>(c);
  *per = static_cast<uint32_t>(div_up(numel, c));
}

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT size_t ksq_moe_align_capacity(size_t numel, size_t E, size_t block_m) {
  if (block_m == 0) return 0;
  return numel + E * (block_m - 1);
}

KSQ_EXPORT size_t ksq_moe_align_scratch_bytes(size_t numel, size_t E) {
  uint32_t chunks, per;
  align_geometry(numel, &chunks, &per);
  size_t bytes = (static_cast<size_t>(chunks) + 1) * E * sizeof(int32_t);
  chunk_geometry(numel, &chunks, &per);
  const size_t parallel = static_cast<size_t>(chunks) * E * sizeof(int32_t);
  return bytes > parallel ? bytes : parallel;
}

KSQ_EXPORT int ksq_moe_align(const void* topk_ids, size_t numel, size_t E, size_t block_m, void* sorted_ids,
                             void* expert_ids, void* num_post_pad, void* scratch, void* stream) {
  const char* fn = "ksq_moe_align";
  if (!sorted_ids || !expert_ids || !num_post_pad || !scratch || (!topk_ids && numel))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (E == 0 || E > 4096) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: expert count %zu outside 1..4096", fn, E);
  if (block_m == 0 || block_m > 1024) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: block_m %zu outside 1..1024", fn, block_m);
  const size_t cap = ksq_moe_align_capacity(numel, E, block_m);
  if (cap > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: too many ids", fn);
  uint32_t chunks, per;
  if (numel >= kParallelAlignFrom) {
    chunk_geometry(numel, &chunks, &per);
    moe_align_count_kernel<<<chunks, kChunkThreads, E * sizeof(int32_t), as_stream(stream)>>>(
        static_cast<const int32_t*>(topk_ids), static_cast<uint32_t>(numel), static_cast<uint32_t>(E),
        static_cast<uint32_t>(cap), static_cast<int32_t*>(sorted_ids), static_cast<int32_t*>(scratch), per);
    moe_align_place_kernel<<<chunks, kChunkThreads, (3 * E + 2 + kChunkThreads) * sizeof(int32_t), as_stream(stream)>>>(
        static_cast<const int32_t*>(topk_ids), static_cast<uint32_t>(numel), static_cast<uint32_t>(E),
        static_cast<uint32_t>(block_m), static_cast<int32_t*>(sorted_ids), static_cast<int32_t*>(expert_ids),
        static_cast<int32_t*>(num_post_pad), static_cast<const int32_t*>(scratch), chunks, per);
    return check_launch(fn);
  }
  if (numel <= 1024 && div_up(numel, 64) * E <= 12288) {  // one id per thread, counters in LDS (at most 48 KiB of them)
    const size_t small_lds = (div_up(numel, 64) * E + 2 * (E + 1)) * sizeof(int32_t);
    const unsigned threads = numel <= 256 ? 256u : 1024u;
    moe_align_small_kernel<<<1, threads, small_lds, as_stream(stream)>>>(
        static_cast<const int32_t*>(topk_ids), static_cast<uint32_t>(numel), static_cast<uint32_t>(E),
        static_cast<uint32_t>(block_m), static_cast<uint32_t>(cap), static_cast<int32_t*>(sorted_ids),
        static_cast<int32_t*>(expert_ids), static_cast<int32_t*>(num_post_pad));
    return check_launch(fn);
  }
  align_geometry(numel, &chunks, &per);
  const size_t lds = 2 * (E + 1) * sizeof(int32_t);
  moe_align_kernel<<<1, kAlignThreads, lds, as_stream(stream)>>>(
      static_cast<const int32_t*>(topk_ids), static_cast<uint32_t>(numel), static_cast<uint32_t>(E),
      static_cast<uint32_t>(block_m), static_cast<uint32_t>(cap), static_cast<int32_t*>(sorted_ids),
      static_cast<int32_t*>(expert_ids), static_cast<int32_t*>(num_post_pad), static_cast<int32_t*>(scratch), chunks,
      per);
  return check_launch(fn);
}

KSQ_EXPORT int ksq_moe_topk_softmax(const void* gating, void* topk_w, void* topk_ids, size_t tokens, size_t E,
                                    size_t top_k, int norm_topk_prob, float routed_scaling_factor, int dtype,
                                    void* stream) {
  const char* fn = "ksq_moe_topk_softmax";
  if (!gating || !topk_w || !topk_ids) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (E == 0 || E > 1024 || top_k == 0 || top_k > 32 || top_k > E)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need 1 <= top_k <= min(32, E) and E <= 1024", fn);
  if (tokens == 0) return KSQ_OK;
  if (tokens > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: too many tokens", fn);
  const unsigned blocks = static_cast<unsigned>(div_up(tokens, 4));
  float* w = static_cast<float*>(topk_w);
  int32_t* ids = static_cast<int32_t*>(topk_ids);
  const uint32_t t = static_cast<uint32_t>(tokens), e = static_cast<uint32_t>(E), k = static_cast<uint32_t>(top_k);
  hipStream_t st = as_stream(stream);
#define KSQ_ROUTE(LOAD_)                                                                                             \
  do {                                                                                                              \
    if (E <= 256)                                                                                                   \
      topk_softmax_kernel<LOAD_, 4><<<blocks, 256, 0, st>>>(gating, w, ids, t, e, k, norm_topk_prob, routed_scaling_factor);  \
    else                                                                                                            \
      topk_softmax_kernel<LOAD_, 16><<<blocks, 256, 0, st>>>(gating, w, ids, t, e, k, norm_topk_prob, routed_scaling_factor); \
  } while (0)
  if (dtype == KSQ_F32) KSQ_ROUTE(LoadF32);
  else if (dtype == KSQ_F16) KSQ_ROUTE(Load16<F16>);
  else if (dtype == KSQ_BF16) KSQ_ROUTE(Load16<BF16>);
  else return fail(KSQ_ERR_UNSUPPORTED, "%s: unknown dtype %d", fn, dtype);
#undef KSQ_ROUTE
  return check_launch(fn);
}

KSQ_EXPORT int ksq_moe_grouped_topk(const void* gating, const void* e_bias, void* topk_w, void* topk_ids, size_t tokens,
                                    size_t E, size_t top_k, size_t num_expert_group, size_t topk_group, int scoring,
                                    int renormalize, float routed_scaling_factor, int dtype, void* stream) {
  const char* fn = "ksq_moe_grouped_topk";
  if (!gating || !topk_w || !topk_ids) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (E == 0 || E > 1024 || top_k == 0 || top_k > 32 || top_k > E)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need 1 <= top_k <= min(32, E) and E <= 1024", fn);
  if (num_expert_group == 0 || num_expert_group > 64 || E % num_expert_group != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need 1 <= num_expert_group <= 64 dividing E", fn);
  if (topk_group == 0 || topk_group > num_expert_group)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need 1 <= topk_group <= num_expert_group", fn);
  const size_t per_group = E / num_expert_group;
  if (e_bias && per_group < 2)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: with a bias a group is ranked by its two best experts and needs two", fn);
  if (top_k > topk_group * per_group)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: top_k %zu exceeds the %zu experts of the kept groups", fn, top_k, topk_group * per_group);
  if (scoring != KSQ_SCORE_SOFTMAX && scoring != KSQ_SCORE_SIGMOID)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: unknown scoring function %d", fn, scoring);
  if (tokens == 0) return KSQ_OK;
  if (tokens > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: too many tokens", fn);
  const unsigned blocks = static_cast<unsigned>(div_up(tokens, 4));
  const size_t lds = 4 * E * sizeof(float);
  float* w = static_cast<float*>(topk_w);
  int32_t* ids = static_cast<int32_t*>(topk_ids);
  const float* b = static_cast<const float*>(e_bias);
  const uint32_t t = static_cast<uint32_t>(tokens), e = static_cast<uint32_t>(E), k = static_cast<uint32_t>(top_k);
  const uint32_t g = static_cast<uint32_t>(num_expert_group), kg = static_cast<uint32_t>(topk_group);
  const int sig = scoring == KSQ_SCORE_SIGMOID;
  hipStream_t st = as_stream(stream);
#define KSQ_ROUTE(LOAD_)                                                                                                         \
  do {                                                                                                                          \
    if (E <= 256)                                                                                                               \
      grouped_topk_kernel<LOAD_, 4><<<blocks, 256, lds, st>>>(gating, b, w, ids, t, e, k, g, kg, sig, renormalize, routed_scaling_factor);  \
    else                                                                                                                        \
      grouped_topk_kernel<LOAD_, 16><<<blocks, 256, lds, st>>>(gating, b, w, ids, t, e, k, g, kg, sig, renormalize, routed_scaling_factor); \
  } while (0)
  if (dtype == KSQ_F32) KSQ_ROUTE(LoadF32);
  else if (dtype == KSQ_F16) KSQ_ROUTE(Load16<F16>);
  else if (dtype == KSQ_BF16) KSQ_ROUTE(Load16<BF16>);
  else return fail(KSQ_ERR_UNSUPPORTED, "%s: unknown dtype %d", fn, dtype);
#undef KSQ_ROUTE
  return check_launch(fn);
}

KSQ_EXPORT int ksq_moe_silu_mul(const void* x, void* out, size_t rows, size_t inter, int dtype, void* stream) {
  const char* fn = "ksq_moe_silu_mul";
  if (!x || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (!aligned16(x) || !aligned16(out)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
  if (inter == 0 || inter % 8 != 0 || inter > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: inter must be a positive multiple of 8", fn);
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  if (rows == 0) return KSQ_OK;
  // a workgroup's 256 threads: 2^log2p column pieces (of 8 elements) by 256 >> log2p rows
  const size_t pieces = inter / 8;
  uint32_t log2p = 0;
  while (log2p < 8 && (size_t(1) << log2p) < pieces) ++log2p;
  const size_t row_blocks = div_up(rows, size_t(256) >> log2p);
  const size_t gy = row_blocks < 32768 ? row_blocks : 32768;
  const size_t gz = div_up(row_blocks, gy);
  if (gz > 65535) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  const dim3 grid(static_cast<unsigned>(div_up(pieces, size_t(1) << log2p)), static_cast<unsigned>(gy), static_cast<unsigned>(gz));
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  uint16_t* op = static_cast<uint16_t*>(out);
  if (dtype == KSQ_F16)
    silu_mul_kernel<F16><<<grid, 256, 0, as_stream(stream)>>>(xp, op, rows, static_cast<uint32_t>(inter), log2p);
  else
    silu_mul_kernel<BF16><<<grid, 256, 0, as_stream(stream)>>>(xp, op, rows, static_cast<uint32_t>(inter), log2p);
  return check_launch(fn);
}

KSQ_EXPORT int ksq_moe_sum(const void* in, void* out, size_t tokens, size_t topk, size_t d, int dtype, void* stream) {
  const char* fn = "ksq_moe_sum";
  if (!in || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (!aligned16(in) || !aligned16(out)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
  if (d == 0 || d % 8 != 0 || d > 0x7fffffffull || topk == 0 || topk > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: d must be a positive multiple of 8 and topk positive", fn);
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  if (tokens == 0) return KSQ_OK;
  const size_t blocks = div_up(tokens * (d / 8), 256);
  if (blocks > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  const uint16_t* ip = static_cast<const uint16_t*>(in);
  uint16_t* op = static_cast<uint16_t*>(out);
  if (dtype == KSQ_F16)
    moe_sum_kernel<F16><<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(ip, op, tokens, static_cast<uint32_t>(topk), static_cast<uint32_t>(d));
  else
    moe_sum_kernel<BF16><<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(ip, op, tokens, static_cast<uint32_t>(topk), static_cast<uint32_t>(d));
  return check_launch(fn);
}
