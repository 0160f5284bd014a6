// Load-time repack between checkpoint int4 layouts and the CDNA4 tile layout described in ksq.h.
// Pure nibble permutations: bit-exact and exactly invertible.
#include "ksq_common.h"

namespace ksq {
namespace {

// AWQ: logical column 8j+i sits in nibble kAwqNib[i] of word j (S/models/quant/cutlass_utils.cpp:12-38)
__device__ __forceinline__ int awq_nibble(int i) {
  // {0,4,1,5,2,6,3,7}
  return ((i & 1) << 2) | (i >> 1);
}
// position of code (k % 8 == j) inside a packed dword: even j in nibbles 0..3, odd j in nibbles 4..7
__device__ __forceinline__ int packed_nibble(int j) { return ((j & 1) << 2) | (j >> 1); }

struct Geometry {
  size_t E, K, N;
  size_t k_tiles, n_tiles;
};

// packed dword index of element (e, k, n)
__device__ __forceinline__ size_t packed_dword(const Geometry& g, size_t e, size_t k, size_t n) {
  size_t tile = (e * g.n_tiles + n / 16) * g.k_tiles + k / 128;
  size_t lane = ((k % 32) / 8) * 16 + (n % 16);
  size_t d = (k % 128) / 32;
  return tile * 256 + lane * 4 + d;
}

template <int SRC>
__global__ void __launch_bounds__(256) repack_weight_kernel(const void* __restrict__ src_v,
                                                            uint32_t* __restrict__ dst, Geometry g) {
  size_t o = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  size_t total = g.E * g.K * g.N / 8;
  if (o >= total) return;
  size_t tile = o / 256;
  int within = static_cast<int>(o % 256);
  int lane = within / 4, d = within % 4;
  size_t kt = tile % g.k_tiles;
  size_t nt = (tile / g.k_tiles) % g.n_tiles;
  size_t e = tile / (g.k_tiles * g.n_tiles);
  size_t n = nt * 16 + (lane % 16);
  size_t kbase = kt * 128 + d * 32 + (lane / 16) * 8;

  uint32_t codes[8];
  if (SRC == KSQ_SRC_GPTQ) {
    const uint32_t* src = static_cast<const uint32_t*>(src_v);
    uint32_t w = src[(e * (g.K / 8) + kbase / 8) * g.N + n];
#pragma unroll
    for (int j = 0; j < 8; ++j) codes[j] = (w >> (4 * j)) & 15u;
  } else if (SRC == KSQ_SRC_MOE_NK) {
    const uint8_t* src = static_cast<const uint8_t*>(src_v);
    uint32_t w = *reinterpret_cast<const uint32_t*>(src + (e * g.N + n) * (g.K / 2) + kbase / 2);
#pragma unroll
    for (int j = 0; j < 8; ++j) codes[j] = (w >> (4 * j)) & 15u;
  } else if (SRC == KSQ_SRC_AWQ) {
    const uint32_t* src = static_cast<const uint32_t*>(src_v);
    int sh = 4 * awq_nibble(static_cast<int>(n % 8));
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t w = src[(e * g.K + kbase + j) * (g.N / 8) + n / 8];
      codes[j] = (w >> sh) & 15u;
    }
  } else {  // KSQ_SRC_INT4X2_KN
    const uint8_t* src = static_cast<const uint8_t*>(src_v);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t b = src[(e * g.K + kbase + j) * (g.N / 2) + n / 2];
      codes[j] = (((n & 1) ? (b >> 4) : b) & 15u) ^ 8u;
    }
  }
  uint32_t out = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) out |= codes[j] << (4 * packed_nibble(j));
  dst[o] = out;
}

// GPTQ act-order: packed row k takes checkpoint row perm[k] (perm = stable argsort of g_idx, so that the rows of a
// quantization group become adjacent); E = 1
__global__ void __launch_bounds__(256) repack_act_order_kernel(const uint32_t* __restrict__ src,
                                                               const int32_t* __restrict__ perm,
                                                               uint32_t* __restrict__ dst, Geometry g) {
  size_t o = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  size_t total = g.K * g.N / 8;
  if (o >= total) return;
  size_t tile = o / 256;
  int within = static_cast<int>(o % 256);
  int lane = within / 4, d = within % 4;
  size_t kt = tile % g.k_tiles;
  size_t nt = tile / g.k_tiles;
  size_t n = nt * 16 + (lane % 16);
  size_t kbase = kt * 128 + d * 32 + (lane / 16) * 8;
  uint32_t out = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    uint32_t row = static_cast<uint32_t>(perm[kbase + j]);
    row = row < g.K ? row : static_cast<uint32_t>(g.K - 1);  // the host checks perm; never read outside the weight
    const uint32_t w = src[static_cast<size_t>(row / 8) * g.N + n];
    out |= ((w >> (4 * (row % 8))) & 15u) << (4 * packed_nibble(j));
  }
  dst[o] = out;
}

// The same for a K range cut out of an act-order checkpoint (a tensor-parallel rank's rows): the packed weight has
// K_dst >= K_src rows, packed row j takes checkpoint row rows[j], and a row index outside [0, K_src) stands for a padding
// row that must contribute nothing: it takes code 8, the symmetric zero point.
__global__ void __launch_bounds__(256) repack_rows_kernel(const uint32_t* __restrict__ src, const int32_t* __restrict__ rows,
                                                          uint32_t* __restrict__ dst, uint32_t K_src, Geometry g) {
  size_t o = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  size_t total = g.K * g.N / 8;
  if (o >= total) return;
  size_t tile = o / 256;
  int within = static_cast<int>(o % 256);
  int lane = within / 4, d = within % 4;
  size_t kt = tile % g.k_tiles;
  size_t nt = tile / g.k_tiles;
  size_t n = nt * 16 + (lane % 16);
  size_t kbase = kt * 128 + d * 32 + (lane / 16) * 8;
  uint32_t out = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t row = static_cast<uint32_t>(rows[kbase + j]);
    uint32_t code = 8u;
    if (row < K_src) code = (src[static_cast<size_t>(row / 8) * g.N + n] >> (4 * (row % 8))) & 15u;
    out |= code << (4 * packed_nibble(j));
  }
  dst[o] = out;
}

// out[r, j] = x[r, idx[j]] for j < k_out, 0 where idx[j] lies outside [0, k_in): the activation side of the above
__global__ void __launch_bounds__(256) gather_columns_kernel(const uint16_t* __restrict__ x, const int32_t* __restrict__ idx,
                                                             uint16_t* __restrict__ out, size_t m, uint32_t k_in, uint32_t k_out) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;  // one thread per 2 output columns
  const size_t per_row = k_out / 2;
  if (i >= m * per_row) return;
  const size_t r = i / per_row;
  const uint32_t c = static_cast<uint32_t>(i % per_row) * 2;
  const uint32_t p0 = static_cast<uint32_t>(idx[c]), p1 = static_cast<uint32_t>(idx[c + 1]);
  const uint16_t* row = x + r * k_in;
  const uint32_t lo = p0 < k_in ? row[p0] : 0u, hi = p1 < k_in ? row[p1] : 0u;
  reinterpret_cast<uint32_t*>(out + r * k_out)[c / 2] = lo | (hi << 16);
}

// out[r, j] = x[r, perm[j]]: the activation side of act-order
__global__ void __launch_bounds__(256) permute_columns_kernel(const uint16_t* __restrict__ x, const int32_t* __restrict__ perm,
                                                              uint16_t* __restrict__ out, size_t m, uint32_t k) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;  // one thread per 2 output columns
  const size_t per_row = k / 2;
  if (i >= m * per_row) return;
  const size_t r = i / per_row;
  const uint32_t c = static_cast<uint32_t>(i % per_row) * 2;
  uint32_t p0 = static_cast<uint32_t>(perm[c]), p1 = static_cast<uint32_t>(perm[c + 1]);
  p0 = p0 < k ? p0 : k - 1;
  p1 = p1 < k ? p1 : k - 1;
  const uint16_t* row = x + r * k;
  reinterpret_cast<uint32_t*>(out + r * k)[c / 2] = static_cast<uint32_t>(row[p0]) | (static_cast<uint32_t>(row[p1]) << 16);
}

// out[s, j] = x[s / top_k, perm[ids[s], j]]: the activation side of act-order for expert stacks, one row per
// (token, slot); slots whose id is not an expert (masked out by an expert map) get row 0's permutation of expert 0 -
// their rows are never read by the grouped GEMM
__global__ void __launch_bounds__(256) moe_permute_columns_kernel(const uint16_t* __restrict__ x, const int32_t* __restrict__ perm,
                                                                  const int32_t* __restrict__ ids, uint16_t* __restrict__ out,
                                                                  size_t numel, uint32_t k, uint32_t top_k, uint32_t E) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;  // one thread per 2 output columns
  const size_t per_row = k / 2;
  if (i >= numel * per_row) return;
  const size_t s = i / per_row;
  const uint32_t c = static_cast<uint32_t>(i % per_row) * 2;
  uint32_t e = static_cast<uint32_t>(ids[s]);
  e = e < E ? e : 0;
  const int32_t* pe = perm + static_cast<size_t>(e) * k;
  uint32_t p0 = static_cast<uint32_t>(pe[c]), p1 = static_cast<uint32_t>(pe[c + 1]);
  p0 = p0 < k ? p0 : k - 1;
  p1 = p1 < k ? p1 : k - 1;
  const uint16_t* row = x + (s / top_k) * k;
  reinterpret_cast<uint32_t*>(out + s * k)[c / 2] = static_cast<uint32_t>(row[p0]) | (static_cast<uint32_t>(row[p1]) << 16);
}

// The same two gathers with the source row staged in LDS: one workgroup per output row loads the row with coalesced
// 16-byte loads, then every thread gathers eight output elements from LDS and stores them as 16 bytes.  (The kernels
// above fetch 2-byte elements from scattered places of the row in memory: 1.7 TB/s where this form is bound by the
// traffic.)  k % 8 == 0 and k * 2 bytes of LDS; ids == nullptr is the dense form (row r reads x[r], one perm).
__global__ void __launch_bounds__(256) permute_row_lds_kernel(const uint16_t* __restrict__ x, const int32_t* __restrict__ perm,
                                                              const int32_t* __restrict__ ids, uint16_t* __restrict__ out,
                                                              uint32_t k, uint32_t top_k, uint32_t E) {
  extern __shared__ __attribute__((aligned(16))) uint16_t row_lds[];
  const size_t s = blockIdx.x;
  const uint16_t* row = x + (ids ? s / top_k : s) * k;
  const int32_t* pe = perm;
  if (ids) {
    uint32_t e = static_cast<uint32_t>(ids[s]);
    e = e < E ? e : 0;
    pe += static_cast<size_t>(e) * k;
  }
  for (uint32_t c = threadIdx.x * 8; c < k; c += 256 * 8)
    *reinterpret_cast<u32x4*>(row_lds + c) = *reinterpret_cast<const u32x4*>(row + c);
  __syncthreads();
  for (uint32_t c = threadIdx.x * 8; c < k; c += 256 * 8) {
    const u32x4 p0 = *reinterpret_cast<const u32x4*>(pe + c);
    const u32x4 p1 = *reinterpret_cast<const u32x4*>(pe + c + 4);
    uint32_t v[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t a = p0[j] < k ? p0[j] : k - 1, b = p1[j] < k ? p1[j] : k - 1;
      v[j] = row_lds[a];
      v[4 + j] = row_lds[b];
    }
    u32x4 o;
    o.x = v[0] | (v[1] << 16);
    o.y = v[2] | (v[3] << 16);
    o.z = v[4] | (v[5] << 16);
    o.w = v[6] | (v[7] << 16);
    *reinterpret_cast<u32x4*>(out + s * k + c) = o;
  }
}

// true when the LDS form serves the call: rows of whole 16-byte pieces, aligned, at most 64 KiB, and enough rows to
// give every CU a workgroup (with few rows the direct form spreads a row over many workgroups and is faster)
inline bool permute_in_lds(const void* x, const void* perm, const void* out, size_t rows, size_t k) {
  return rows >= 256 && rows <= 0x7fffffffull && k % 8 == 0 && k * 2 <= 65536 && aligned16(x) && aligned16(perm) &&
         aligned16(out);
}

// FP8 weights [E, N, K] (checkpoint, row-major) <-> 2 KiB fragments of 16 rows x 128 k, fragment (e, n/16, k/128) at
// ((e*N/16 + n/16)*(K/128) + k/128): half h, then lane l = 16*((k%128)/32) + n%16, then the 16 bytes
// k%32 in [16h, 16h+16) - the two 16-byte halves of the lane's operand of v_mfma_f32_16x16x128_f8f6f4.
// One thread moves 16 bytes; TO_PACKED selects the direction.
template <bool TO_PACKED>
__global__ void __launch_bounds__(256) fp8_repack_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                         size_t E, size_t N, size_t K) {
  const size_t o = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;  // 16-byte piece of the packed tensor
  if (o >= E * N * K / 16) return;
  const size_t KB = K / 128;
  const size_t frag = o / 128;
  const uint32_t within = static_cast<uint32_t>(o % 128);
  const uint32_t h = within / 64, lane = within % 64;
  const size_t kb = frag % KB;
  const size_t nt = (frag / KB) % (N / 16);
  const size_t e = frag / (KB * (N / 16));
  const size_t row = nt * 16 + (lane % 16);
  const size_t kbyte = kb * 128 + (lane / 16) * 32 + h * 16;
  const size_t plain = ((e * N + row) * K + kbyte) / 16;
  if (TO_PACKED) dst[o] = src[plain];
  else dst[plain] = src[o];
}

// one thread per 8 codes of the destination
template <int DST>
__global__ void __launch_bounds__(256) unpack_weight_kernel(const uint32_t* __restrict__ packed,
                                                            void* __restrict__ dst_v, Geometry g) {
  size_t o = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  size_t total = g.E * g.K * g.N / 8;
  if (o >= total) return;
  if (DST == KSQ_SRC_GPTQ || DST == KSQ_SRC_MOE_NK) {
    size_t e, kp, n;
    if (DST == KSQ_SRC_GPTQ) {  // dst word (e, kp, n)
      n = o % g.N;
      kp = (o / g.N) % (g.K / 8);
      e = o / (g.N * (g.K / 8));
    } else {  // dst u32 (e, n, kp)
      kp = o % (g.K / 8);
      n = (o / (g.K / 8)) % g.N;
      e = o / (g.N * (g.K / 8));
    }
    uint32_t w = packed[packed_dword(g, e, kp * 8, n)];
    uint32_t out = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) out |= ((w >> (4 * packed_nibble(j))) & 15u) << (4 * j);
    static_cast<uint32_t*>(dst_v)[o] = out;
  } else {  // AWQ word (e, k, n/8) or four INT4X2 bytes (e, k, n/2 .. +3)
    size_t j8 = o % (g.N / 8);
    size_t k = (o / (g.N / 8)) % g.K;
    size_t e = o / ((g.N / 8) * g.K);
    int sh = 4 * packed_nibble(static_cast<int>(k % 8));
    uint32_t out = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t c = (packed[packed_dword(g, e, k, j8 * 8 + i)] >> sh) & 15u;
      if (DST == KSQ_SRC_AWQ)
        out |= c << (4 * awq_nibble(i));
      else
        out |= (c ^ 8u) << (4 * i);
    }
    static_cast<uint32_t*>(dst_v)[o] = out;
  }
}

// scales: 16-bit elements.  packed index = ((e*n_tiles + n/16)*G + g)*16 + n%16
template <int LAYOUT, bool TO_PACKED>
__global__ void __launch_bounds__(256) scales_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                     size_t E, size_t G, size_t N) {
  size_t o = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (o >= E * G * N) return;
  size_t nn = o % 16;
  size_t gi = (o / 16) % G;
  size_t nt = (o / (16 * G)) % (N / 16);
  size_t e = o / (16 * G * (N / 16));
  size_t n = nt * 16 + nn;
  size_t lin = (LAYOUT == KSQ_SCALE_GN) ? (e * G + gi) * N + n : (e * N + n) * G + gi;
  if (TO_PACKED)
    dst[o] = src[lin];
  else
    dst[lin] = src[o];
}

template <int LAYOUT>
__global__ void __launch_bounds__(256) zeros_pack_kernel(const void* __restrict__ src_v, uint8_t* __restrict__ dst,
                                                         size_t G, size_t N) {
  size_t o = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (o >= G * N) return;
  size_t nn = o % 16;
  size_t gi = (o / 16) % G;
  size_t nt = o / (16 * G);
  size_t n = nt * 16 + nn;
  if (LAYOUT == KSQ_ZERO_AWQ_PACKED) {
    uint32_t w = static_cast<const uint32_t*>(src_v)[gi * (N / 8) + n / 8];
    dst[o] = static_cast<uint8_t>((w >> (4 * awq_nibble(static_cast<int>(n % 8)))) & 15u);
  } else {
    dst[o] = static_cast<const uint8_t*>(src_v)[gi * N + n];
  }
}

// one thread per 8 zero points of the destination
template <int LAYOUT>
__global__ void __launch_bounds__(256) zeros_unpack_kernel(const uint8_t* __restrict__ packed,
                                                           void* __restrict__ dst_v, size_t G, size_t N) {
  size_t o = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (o >= G * N / 8) return;
  size_t j8 = o % (N / 8);
  size_t gi = o / (N / 8);
  uint32_t out = 0;
  for (int i = 0; i < 8; ++i) {
    size_t n = j8 * 8 + i;
    uint32_t z = packed[((n / 16) * G + gi) * 16 + n % 16];
    if (LAYOUT == KSQ_ZERO_AWQ_PACKED)
      out |= (z & 15u) << (4 * awq_nibble(i));
    else
      static_cast<uint8_t*>(dst_v)[gi * N + n] = static_cast<uint8_t>(z);
  }
  if (LAYOUT == KSQ_ZERO_AWQ_PACKED) static_cast<uint32_t*>(dst_v)[o] = out;
}

int check_weight_args(const void* a, const void* b, size_t E, size_t K, size_t N, const char* fn) {
  if (!a || !b) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (!aligned16(a) || !aligned16(b)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
  if (E == 0 || K == 0 || N == 0 || K % 128 != 0 || N % 16 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need E>0, K %% 128 == 0, N %% 16 == 0 (E=%zu K=%zu N=%zu)", fn, E, K, N);
  if (E * K * N / 8 / 256 + 1 > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  return KSQ_OK;
}

int check_group(size_t K, size_t group, const char* fn) {
  if (group != 32 && group != 64 && group != 128)
    return fail(KSQ_ERR_UNSUPPORTED, "%s: group size %zu not in {32,64,128}", fn, group);
  if (K % group) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: K not a multiple of group", fn);
  return KSQ_OK;
}

}  // namespace
}  // namespace ksq

using namespace ksq;

KSQ_EXPORT int ksq_w4a16_repack(const void* src, int src_layout, void* dst, size_t E, size_t K, size_t N,
                                void* stream) {
  if (int rc = check_weight_args(src, dst, E, K, N, "ksq_w4a16_repack")) return rc;
  Geometry g{E, K, N, K / 128, N / 16};
  unsigned blocks = static_cast<unsigned>(div_up(E * K * N / 8, 256));
  hipStream_t s = as_stream(stream);
  uint32_t* d = static_cast<uint32_t*>(dst);
  switch (src_layout) {
    case KSQ_SRC_GPTQ:
      repack_weight_kernel<KSQ_SRC_GPTQ><<<blocks, 256, 0, s>>>(src, d, g);
      break;
    case KSQ_SRC_AWQ:
      repack_weight_kernel<KSQ_SRC_AWQ><<<blocks, 256, 0, s>>>(src, d, g);
      break;
    case KSQ_SRC_MOE_NK:
      repack_weight_kernel<KSQ_SRC_MOE_NK><<<blocks, 256, 0, s>>>(src, d, g);
      break;
    case KSQ_SRC_INT4X2_KN:
      repack_weight_kernel<KSQ_SRC_INT4X2_KN><<<blocks, 256, 0, s>>>(src, d, g);
      break;
    default:
      return fail(KSQ_ERR_INVALID_ARGUMENT, "ksq_w4a16_repack: unknown source layout %d", src_layout);
  }
  return check_launch("ksq_w4a16_repack");
}

KSQ_EXPORT int ksq_w4a16_repack_act_order(const void* src_gptq, const void* perm, void* dst, size_t K, size_t N,
                                          void* stream) {
  const char* fn = "ksq_w4a16_repack_act_order";
  if (int rc = check_weight_args(src_gptq, dst, 1, K, N, fn)) return rc;
  if (!perm || (reinterpret_cast<uintptr_t>(perm) & 3u)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: perm must be a 4-byte aligned pointer", fn);
  Geometry g{1, K, N, K / 128, N / 16};
  unsigned blocks = static_cast<unsigned>(div_up(K * N / 8, 256));
  repack_act_order_kernel<<<blocks, 256, 0, as_stream(stream)>>>(static_cast<const uint32_t*>(src_gptq),
                                                                  static_cast<const int32_t*>(perm),
                                                                  static_cast<uint32_t*>(dst), g);
  return check_launch(fn);
}

static int fp8_repack_common(const void* src, void* dst, size_t E, size_t N, size_t K, void* stream, bool to_packed,
                             const char* fn) {
  if (!src || !dst) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if (!aligned16(src) || !aligned16(dst)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
  if (src == dst) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: cannot repack in place", fn);
  if (E == 0 || N == 0 || K == 0 || K % 128 != 0 || N % 16 != 0)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: need E>0, K %% 128 == 0, N %% 16 == 0 (E=%zu N=%zu K=%zu)", fn, E, N, K);
  const size_t blocks = div_up(E * N * K / 16, 256);
  if (blocks > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  const u32x4* s = static_cast<const u32x4*>(src);
  u32x4* d = static_cast<u32x4*>(dst);
  if (to_packed) fp8_repack_kernel<true><<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(s, d, E, N, K);
  else fp8_repack_kernel<false><<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(s, d, E, N, K);
  return check_launch(fn);
}

KSQ_EXPORT int ksq_fp8_repack_weight(const void* src, void* dst_packed, size_t E, size_t N, size_t K, void* stream) {
  return fp8_repack_common(src, dst_packed, E, N, K, stream, true, "ksq_fp8_repack_weight");
}

KSQ_EXPORT int ksq_fp8_unpack_weight(const void* packed, void* dst, size_t E, size_t N, size_t K, void* stream) {
  return fp8_repack_common(packed, dst, E, N, K, stream, false, "ksq_fp8_unpack_weight");
}

KSQ_EXPORT int ksq_permute_columns(const void* x, const void* perm, void* out, size_t m, size_t k, int dtype,
                                   void* stream) {
  const char* fn = "ksq_permute_columns";
  if (!x || !perm || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if ((reinterpret_cast<uintptr_t>(x) & 1u) || (reinterpret_cast<uintptr_t>(out) & 3u) || (reinterpret_cast<uintptr_t>(perm) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: x must be 2-byte, out and perm 4-byte aligned", fn);
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  if (k == 0 || k % 2 != 0 || k > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k must be positive and even", fn);
  if (x == out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: cannot permute in place", fn);
  if (m == 0) return KSQ_OK;
  if (permute_in_lds(x, perm, out, m, k)) {
    permute_row_lds_kernel<<<static_cast<unsigned>(m), 256, k * 2, as_stream(stream)>>>(
        static_cast<const uint16_t*>(x), static_cast<const int32_t*>(perm), nullptr, static_cast<uint16_t*>(out),
        static_cast<uint32_t>(k), 1u, 1u);
    return check_launch(fn);
  }
  const size_t blocks = div_up(m * (k / 2), 256);
  if (blocks > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  permute_columns_kernel<<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(
      static_cast<const uint16_t*>(x), static_cast<const int32_t*>(perm), static_cast<uint16_t*>(out), m,
      static_cast<uint32_t>(k));
  return check_launch(fn);
}

KSQ_EXPORT int ksq_w4a16_repack_rows(const void* src_gptq, const void* rows, void* dst, size_t K_src, size_t K_dst, size_t N,
                                     void* stream) {
  const char* fn = "ksq_w4a16_repack_rows";
  if (int rc = check_weight_args(src_gptq, dst, 1, K_dst, N, fn)) return rc;
  if (K_src == 0 || K_src % 8 != 0 || K_src > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: K_src must be a positive multiple of 8", fn);
  if (!rows || (reinterpret_cast<uintptr_t>(rows) & 3u)) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: rows must be a 4-byte aligned pointer", fn);
  Geometry g{1, K_dst, N, K_dst / 128, N / 16};
  unsigned blocks = static_cast<unsigned>(div_up(K_dst * N / 8, 256));
  repack_rows_kernel<<<blocks, 256, 0, as_stream(stream)>>>(static_cast<const uint32_t*>(src_gptq), static_cast<const int32_t*>(rows),
                                                             static_cast<uint32_t*>(dst), static_cast<uint32_t>(K_src), g);
  return check_launch(fn);
}

KSQ_EXPORT int ksq_gather_columns(const void* x, const void* idx, void* out, size_t m, size_t k_in, size_t k_out, int dtype,
                                  void* stream) {
  const char* fn = "ksq_gather_columns";
  if (!x || !idx || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if ((reinterpret_cast<uintptr_t>(x) & 1u) || (reinterpret_cast<uintptr_t>(out) & 3u) || (reinterpret_cast<uintptr_t>(idx) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: x must be 2-byte, out and idx 4-byte aligned", fn);
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  if (k_in == 0 || k_out == 0 || k_out % 2 != 0 || k_in > 0x7fffffffull || k_out > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k_in must be positive, k_out positive and even", fn);
  if (x == out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: cannot gather in place", fn);
  if (m == 0) return KSQ_OK;
  const size_t blocks = div_up(m * (k_out / 2), 256);
  if (blocks > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  gather_columns_kernel<<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(
      static_cast<const uint16_t*>(x), static_cast<const int32_t*>(idx), static_cast<uint16_t*>(out), m,
      static_cast<uint32_t>(k_in), static_cast<uint32_t>(k_out));
  return check_launch(fn);
}

KSQ_EXPORT int ksq_moe_permute_columns(const void* x, const void* perm, const void* topk_ids, void* out, size_t numel,
                                       size_t k, size_t top_k, size_t E, int dtype, void* stream) {
  const char* fn = "ksq_moe_permute_columns";
  if (!x || !perm || !topk_ids || !out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: null pointer", fn);
  if ((reinterpret_cast<uintptr_t>(x) & 1u) || (reinterpret_cast<uintptr_t>(out) & 3u) ||
      (reinterpret_cast<uintptr_t>(perm) & 3u) || (reinterpret_cast<uintptr_t>(topk_ids) & 3u))
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: x must be 2-byte, out, perm and topk_ids 4-byte aligned", fn);
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  if (k == 0 || k % 2 != 0 || k > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: k must be positive and even", fn);
  if (top_k == 0 || E == 0 || top_k > 0x7fffffffull || E > 0x7fffffffull)
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: top_k and E must be positive", fn);
  if (x == out) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: cannot permute in place", fn);
  if (numel == 0) return KSQ_OK;
  if (permute_in_lds(x, perm, out, numel, k)) {
    permute_row_lds_kernel<<<static_cast<unsigned>(numel), 256, k * 2, as_stream(stream)>>>(
        static_cast<const uint16_t*>(x), static_cast<const int32_t*>(perm), static_cast<const int32_t*>(topk_ids),
        static_cast<uint16_t*>(out), static_cast<uint32_t>(k), static_cast<uint32_t>(top_k), static_cast<uint32_t>(E));
    return check_launch(fn);
  }
  const size_t blocks = div_up(numel * (k / 2), 256);
  if (blocks > 0x7fffffffull) return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: tensor too large", fn);
  moe_permute_columns_kernel<<<static_cast<unsigned>(blocks), 256, 0, as_stream(stream)>>>(
      static_cast<const uint16_t*>(x), static_cast<const int32_t*>(perm), static_cast<const int32_t*>(topk_ids),
      static_cast<uint16_t*>(out), numel, static_cast<uint32_t>(k), static_cast<uint32_t>(top_k), static_cast<uint32_t>(E));
  return check_launch(fn);
}

KSQ_EXPORT int ksq_w4a16_unpack(const void* packed, int dst_layout, void* dst, size_t E, size_t K, size_t N,
                                void* stream) {
  if (int rc = check_weight_args(packed, dst, E, K, N, "ksq_w4a16_unpack")) return rc;
  Geometry g{E, K, N, K / 128, N / 16};
  unsigned blocks = static_cast<unsigned>(div_up(E * K * N / 8, 256));
  hipStream_t s = as_stream(stream);
  const uint32_t* p = static_cast<const uint32_t*>(packed);
  switch (dst_layout) {
    case KSQ_SRC_GPTQ:
      unpack_weight_kernel<KSQ_SRC_GPTQ><<<blocks, 256, 0, s>>>(p, dst, g);
      break;
    case KSQ_SRC_AWQ:
      unpack_weight_kernel<KSQ_SRC_AWQ><<<blocks, 256, 0, s>>>(p, dst, g);
      break;
    case KSQ_SRC_MOE_NK:
      unpack_weight_kernel<KSQ_SRC_MOE_NK><<<blocks, 256, 0, s>>>(p, dst, g);
      break;
    case KSQ_SRC_INT4X2_KN:
      unpack_weight_kernel<KSQ_SRC_INT4X2_KN><<<blocks, 256, 0, s>>>(p, dst, g);
      break;
    default:
      return fail(KSQ_ERR_INVALID_ARGUMENT, "ksq_w4a16_unpack: unknown destination layout %d", dst_layout);
  }
  return check_launch("ksq_w4a16_unpack");
}

static int scales_common(const void* src, int layout, void* dst, size_t E, size_t K, size_t N, size_t group, int dtype,
                         void* stream, bool to_packed, const char* fn) {
  if (int rc = check_weight_args(src, dst, E, K, N, fn)) return rc;
  if (int rc = check_group(K, group, fn)) return rc;
  if (dtype != KSQ_F16 && dtype != KSQ_BF16) return fail(KSQ_ERR_UNSUPPORTED, "%s: dtype must be f16 or bf16", fn);
  size_t G = K / group;
  unsigned blocks = static_cast<unsigned>(div_up(E * G * N, 256));
  hipStream_t s = as_stream(stream);
  const uint16_t* a = static_cast<const uint16_t*>(src);
  uint16_t* b = static_cast<uint16_t*>(dst);
  if (layout == KSQ_SCALE_GN) {
    if (to_packed)
      scales_kernel<KSQ_SCALE_GN, true><<<blocks, 256, 0, s>>>(a, b, E, G, N);
    else
      scales_kernel<KSQ_SCALE_GN, false><<<blocks, 256, 0, s>>>(a, b, E, G, N);
  } else if (layout == KSQ_SCALE_NG) {
    if (to_packed)
      scales_kernel<KSQ_SCALE_NG, true><<<blocks, 256, 0, s>>>(a, b, E, G, N);
    else
      scales_kernel<KSQ_SCALE_NG, false><<<blocks, 256, 0, s>>>(a, b, E, G, N);
  } else {
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: unknown scale layout %d", fn, layout);
  }
  return check_launch(fn);
}

KSQ_EXPORT int ksq_w4a16_repack_scales(const void* src, int src_layout, void* dst, size_t E, size_t K, size_t N,
                                       size_t group, int dtype, void* stream) {
  return scales_common(src, src_layout, dst, E, K, N, group, dtype, stream, true, "ksq_w4a16_repack_scales");
}

KSQ_EXPORT int ksq_w4a16_unpack_scales(const void* packed, int dst_layout, void* dst, size_t E, size_t K, size_t N,
                                       size_t group, int dtype, void* stream) {
  return scales_common(packed, dst_layout, dst, E, K, N, group, dtype, stream, false, "ksq_w4a16_unpack_scales");
}

KSQ_EXPORT int ksq_w4a16_repack_zeros(const void* src, int src_layout, void* dst, size_t K, size_t N, size_t group,
                                      void* stream) {
  const char* fn = "ksq_w4a16_repack_zeros";
  if (int rc = check_weight_args(src, dst, 1, K, N, fn)) return rc;
  if (int rc = check_group(K, group, fn)) return rc;
  size_t G = K / group;
  unsigned blocks = static_cast<unsigned>(div_up(G * N, 256));
  hipStream_t s = as_stream(stream);
  if (src_layout == KSQ_ZERO_AWQ_PACKED)
    zeros_pack_kernel<KSQ_ZERO_AWQ_PACKED><<<blocks, 256, 0, s>>>(src, static_cast<uint8_t*>(dst), G, N);
  else if (src_layout == KSQ_ZERO_U8_GN)
    zeros_pack_kernel<KSQ_ZERO_U8_GN><<<blocks, 256, 0, s>>>(src, static_cast<uint8_t*>(dst), G, N);
  else
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: unknown zero-point layout %d", fn, src_layout);
  return check_launch(fn);
}

KSQ_EXPORT int ksq_w4a16_unpack_zeros(const void* packed, int dst_layout, void* dst, size_t K, size_t N, size_t group,
                                      void* stream) {
  const char* fn = "ksq_w4a16_unpack_zeros";
  if (int rc = check_weight_args(packed, dst, 1, K, N, fn)) return rc;
  if (int rc = check_group(K, group, fn)) return rc;
  size_t G = K / group;
  unsigned blocks = static_cast<unsigned>(div_up(G * N / 8, 256));
  hipStream_t s = as_stream(stream);
  if (dst_layout == KSQ_ZERO_AWQ_PACKED)
    zeros_unpack_kernel<KSQ_ZERO_AWQ_PACKED><<<blocks, 256, 0, s>>>(static_cast<const uint8_t*>(packed), dst, G, N);
  else if (dst_layout == KSQ_ZERO_U8_GN)
    zeros_unpack_kernel<KSQ_ZERO_U8_GN><<<blocks, 256, 0, s>>>(static_cast<const uint8_t*>(packed), dst, G, N);
  else
    return fail(KSQ_ERR_INVALID_ARGUMENT, "%s: unknown zero-point layout %d", fn, dst_layout);
  return check_launch(fn);
}
