/*
 * CPU oracle for the quantized-GEMM path of KsanaLLM.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the algorithms of the
 * reference's quantized matmul path so that the HIP library can be checked against
 * them.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load it; the product library never links or calls it.
 *
 * Path shorthands used in citations:
 *   S/ = src/ksana_llm/      K/ = 3rdparty/LLM_kernels/csrc/kernels/nvidia/
 *
 * Pinning status of each function (what fixes it besides this restatement):
 *   f16/bf16/e4m3 converters ....... exhaustive decode tables vs torch CPU casts, RNE tie cases
 *   gptq_unpack / awq_unpack ........ 0x66666666 -> 0xEE known answer (S/models/quant/cutlass_utils_test.cpp:80-108),
 *                                     cross-check vs Marlin repack vectors below
 *   marlin_gptq_repack / awq_repack . arange golden words (S/models/quant/marlin_utils_test.cpp:29-91)
 *   marlin_awq_zero_points .......... arange golden words (marlin_utils_test.cpp:149-173)
 *   w4a16_dequant / gemm ............ all-zero codes -> -8 (S/models/quant/quant_int4_weight_test.cpp:259-287),
 *                                     float64 numpy matmul on tiny shapes
 *   fp8_group_quant ................. x=i/100 known answer (K/others/sglang/main/quantization/fp8/
 *                                     per_token_group_quant_test.cu:77-98), closed-form scale checks
 *   fp8_group_quant(fuse_silu_mul) .. PARITY UNPINNED at bit level: the reference uses NVIDIA tanh.approx.f32
 *                                     (per_token_group_quant.cu:65-76); restated here with tanhf
 *   fp8_blockwise_gemm .............. numpy float64 block-scaled matmul on tiny shapes; restates
 *                                     K/blockwise_gemm/blockwise_gemm_test.cu:138-177
 *   moe_align ....................... worked example in K/moe_utils/moe_utils.cu:150-156, invariants
 *   silu_mul / moe_sum .............. closed forms (K/moe_utils/moe_utils.cu:597-606,549-562)
 *   moe_gemm ........................ equals the dense dequantize-then-multiply of each expert's rows
 *   moe_topk_softmax ................ torch softmax + topk
 *   moe_grouped_topk ................ the published DeepSeek-V2/V3 formula in torch tensor ops, and the reference's own
 *                                     host implementation compiled from the reference tree (oracle/_ref)
 *   fp8_channel_quant ............... torch float8_e4m3fn conversion, every rounding boundary
 *   fp8_tensor_gemm ................. torch fp32 matmul of the decoded operands
 *   w4a8_unpack_int4 ................ hand-written known answers of the sign-extending nibble split
 *                                     (K/others/tensorrt-llm/dev/thop/finegrained_mixed_dtype_gemm_thop_test.cu:53-80)
 *   w4a8_static_quant ............... torch float8_e4m3fn conversion of the fp32 quotient
 *   w4a8_group_sums ................. numpy float64 sums of the decoded values
 *   w4a8_gemm ....................... torch float64 matmul of the reference test's own formula
 *                                     (finegrained_mixed_dtype_gemm_thop_test.cu:186-206) on the decoded operands
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define KSQO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------------
 * Scalar format converters
 * ---------------------------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

KSQO_API float ksqo_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    float v = (float)man * (1.0f / 16777216.0f); /* man * 2^-24 */
    return (sign ? -v : v);
  }
  if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even float -> IEEE binary16 */
KSQO_API uint16_t ksqo_f32_to_f16(float f) {
  uint32_t x = f32_bits(f);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
  }
  if (ax >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x38800000u) { /* subnormal half or zero: value * 2^24 rounded to integer */
    float af = bits_f32(ax);
    float scaled = af * 16777216.0f;
    /* rintf uses the current rounding mode = nearest even */
    uint32_t m = (uint32_t)rintf(scaled);
    return (uint16_t)(sign | m);
  }
  uint32_t e = (ax >> 23) - 112u;
  uint32_t m = ax & 0x7fffffu;
  uint32_t h = (e << 10) | (m >> 13);
  uint32_t rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}

KSQO_API float ksqo_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

KSQO_API uint16_t ksqo_f32_to_bf16(float f) {
  uint32_t x = f32_bits(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

/* OCP e4m3fn decode: bias 7, no inf, 0x7f/0xff = NaN, max 448.
 * Same table as the reference's test decoder, S/kernels/nvidia/kernel_wrapper_test.cpp:87-134. */
KSQO_API float ksqo_e4m3_to_f32(uint8_t c) {
  uint32_t s = c >> 7, e = (c >> 3) & 0xf, m = c & 7;
  float v;
  if (e == 15 && m == 7) return bits_f32(0x7fc00000u | (s << 31));
  if (e == 0)
    v = (float)m * 0.001953125f; /* m * 2^-9 */
  else
    v = ldexpf(1.0f + (float)m / 8.0f, (int)e - 7);
  return s ? -v : v;
}

/* float -> e4m3fn, round-to-nearest-even, saturate-to-finite (+-448), NaN -> 0x7f | sign.
 * Semantics of __nv_cvt_float2_to_fp8x2(x, __NV_SATFINITE, __NV_E4M3) as used at
 * K/others/sglang/main/quantization/fp8/per_token_group_quant.cu:199-207. */
KSQO_API uint8_t ksqo_f32_to_e4m3(float f) {
  uint32_t x = f32_bits(f);
  uint8_t sign = (uint8_t)((x >> 24) & 0x80u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
  float a = bits_f32(ax);
  if (a >= 448.0f) return (uint8_t)(sign | 0x7eu); /* [448,464] rounds to 448 (even mantissa), above saturates */
  if (a < 0.015625f) { /* below 2^-6: subnormal grid of 2^-9 */
    uint32_t m = (uint32_t)rintf(a * 512.0f);
    return (uint8_t)(sign | m); /* m == 8 encodes 2^-6 correctly (exp=1, man=0) */
  }
  int e;
  float fr = frexpf(a, &e); /* a = fr * 2^e, fr in [0.5,1) */
  /* a = (2*fr) * 2^(e-1); mantissa grid 1/8 */
  float scaled = fr * 16.0f; /* in [8,16) */
  uint32_t q = (uint32_t)rintf(scaled);
  int exp = e - 1;
  if (q == 16) {
    q = 8;
    exp += 1;
  }
  uint32_t code = ((uint32_t)(exp + 7) << 3) | (q - 8);
  if (code > 0x7eu) code = 0x7eu;
  return (uint8_t)(sign | code);
}

/* bulk helpers for the python side */
KSQO_API void ksqo_f16_to_f32_n(const uint16_t* h, float* f, size_t n) {
  for (size_t i = 0; i < n; ++i) f[i] = ksqo_f16_to_f32(h[i]);
}
KSQO_API void ksqo_f32_to_f16_n(const float* f, uint16_t* h, size_t n) {
  for (size_t i = 0; i < n; ++i) h[i] = ksqo_f32_to_f16(f[i]);
}
KSQO_API void ksqo_bf16_to_f32_n(const uint16_t* h, float* f, size_t n) {
  for (size_t i = 0; i < n; ++i) f[i] = ksqo_bf16_to_f32(h[i]);
}
KSQO_API void ksqo_f32_to_bf16_n(const float* f, uint16_t* h, size_t n) {
  for (size_t i = 0; i < n; ++i) h[i] = ksqo_f32_to_bf16(f[i]);
}
KSQO_API void ksqo_e4m3_to_f32_n(const uint8_t* c, float* f, size_t n) {
  for (size_t i = 0; i < n; ++i) f[i] = ksqo_e4m3_to_f32(c[i]);
}
KSQO_API void ksqo_f32_to_e4m3_n(const float* f, uint8_t* c, size_t n) {
  for (size_t i = 0; i < n; ++i) c[i] = ksqo_f32_to_e4m3(f[i]);
}

/* dtype tags shared with the C-ABI of the HIP library */
enum { KSQO_F16 = 0, KSQO_BF16 = 1, KSQO_F32 = 2 };

static inline float load_t(const void* p, size_t i, int dtype) {
  if (dtype == KSQO_F16) return ksqo_f16_to_f32(((const uint16_t*)p)[i]);
  if (dtype == KSQO_BF16) return ksqo_bf16_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}
static inline float round_t(float v, int dtype) {
  if (dtype == KSQO_F16) return ksqo_f16_to_f32(ksqo_f32_to_f16(v));
  if (dtype == KSQO_BF16) return ksqo_bf16_to_f32(ksqo_f32_to_bf16(v));
  return v;
}
static inline void store_t(void* p, size_t i, float v, int dtype) {
  if (dtype == KSQO_F16)
    ((uint16_t*)p)[i] = ksqo_f32_to_f16(v);
  else if (dtype == KSQO_BF16)
    ((uint16_t*)p)[i] = ksqo_f32_to_bf16(v);
  else
    ((float*)p)[i] = v;
}

/* ------------------------------------------------------------------------------------------------
 * Checkpoint bit layouts
 * ---------------------------------------------------------------------------------------------- */

/* GPTQ qweight [K/8, N] int32 -> codes [K, N] u8 (0..15); nibble i of word (k/8, n) is row 8*(k/8)+i.
 * S/models/quant/cutlass_utils.cpp:41-50 (CutlassUnpackGPTQ). */
KSQO_API void ksqo_gptq_unpack(const uint32_t* qweight, uint8_t* codes, size_t K, size_t N) {
  for (size_t kp = 0; kp < K / 8; ++kp)
    for (size_t n = 0; n < N; ++n) {
      uint32_t w = qweight[kp * N + n];
      for (int i = 0; i < 8; ++i) codes[(kp * 8 + i) * N + n] = (uint8_t)((w >> (4 * i)) & 0xf);
    }
}

/* inverse of the above (used to build synthetic checkpoints) */
KSQO_API void ksqo_gptq_pack(const uint8_t* codes, uint32_t* qweight, size_t K, size_t N) {
  for (size_t kp = 0; kp < K / 8; ++kp)
    for (size_t n = 0; n < N; ++n) {
      uint32_t w = 0;
      for (int i = 0; i < 8; ++i) w |= (uint32_t)(codes[(kp * 8 + i) * N + n] & 0xf) << (4 * i);
      qweight[kp * N + n] = w;
    }
}

/* AWQ qweight (or qzeros) [R, N/8] int32 -> codes [R, N] u8: column 8j+i is read from nibble
 * {0,4,1,5,2,6,3,7}[i] of word (r, j).
 * S/models/quant/cutlass_utils.cpp:12-38 (CutlassGetReverseOrder + CutlassUnpackAWQ). */
static const int kAwqReverse[8] = {0, 4, 1, 5, 2, 6, 3, 7};

KSQO_API void ksqo_awq_unpack(const uint32_t* q, uint8_t* codes, size_t R, size_t N) {
  for (size_t r = 0; r < R; ++r)
    for (size_t j = 0; j < N / 8; ++j) {
      uint32_t w = q[r * (N / 8) + j];
      for (int i = 0; i < 8; ++i) codes[r * N + j * 8 + i] = (uint8_t)((w >> (4 * kAwqReverse[i])) & 0xf);
    }
}

KSQO_API void ksqo_awq_pack(const uint8_t* codes, uint32_t* q, size_t R, size_t N) {
  for (size_t r = 0; r < R; ++r)
    for (size_t j = 0; j < N / 8; ++j) {
      uint32_t w = 0;
      for (int i = 0; i < 8; ++i) w |= (uint32_t)(codes[r * N + j * 8 + i] & 0xf) << (4 * kAwqReverse[i]);
      q[r * (N / 8) + j] = w;
    }
}

/* [K, N] int8 -> [K, N/2] int8, low nibble = even column.  S/models/quant/cutlass_utils.cpp:53-59. */
KSQO_API void ksqo_pack_int8_to_int4x2(const int8_t* w, int8_t* out, size_t K, size_t N) {
  for (size_t k = 0; k < K; ++k)
    for (size_t j = 0; j < N / 2; ++j) {
      uint8_t lo = (uint8_t)w[k * N + 2 * j] & 0x0f;
      uint8_t hi = (uint8_t)(((uint8_t)w[k * N + 2 * j + 1] & 0x0f) << 4);
      out[k * (N / 2) + j] = (int8_t)(hi | lo);
    }
}

/* MoE expert weight as the loader leaves it: [E, N, K/2] u8, low nibble = even k.
 * S/models/quant/quant_weight.cpp:182-319; in-test dequant S/kernels/nvidia/fused_moe_gptq_awq_test.cpp:119-124. */
KSQO_API void ksqo_moe_unpack(const uint8_t* w, uint8_t* codes /* [E,K,N] */, size_t E, size_t N, size_t K) {
  for (size_t e = 0; e < E; ++e)
    for (size_t n = 0; n < N; ++n)
      for (size_t kk = 0; kk < K / 2; ++kk) {
        uint8_t b = w[(e * N + n) * (K / 2) + kk];
        codes[(e * K + 2 * kk) * N + n] = b & 0xf;
        codes[(e * K + 2 * kk + 1) * N + n] = b >> 4;
      }
}

KSQO_API void ksqo_moe_pack(const uint8_t* codes /* [E,K,N] */, uint8_t* w /* [E,N,K/2] */, size_t E, size_t N,
                            size_t K) {
  for (size_t e = 0; e < E; ++e)
    for (size_t n = 0; n < N; ++n)
      for (size_t kk = 0; kk < K / 2; ++kk) {
        uint8_t lo = codes[(e * K + 2 * kk) * N + n] & 0xf;
        uint8_t hi = codes[(e * K + 2 * kk + 1) * N + n] & 0xf;
        w[(e * N + n) * (K / 2) + kk] = (uint8_t)(lo | (hi << 4));
      }
}

/* ------------------------------------------------------------------------------------------------
 * Marlin repack index maps (test-only oracle; anchors the nibble orders to the reference's vectors)
 * ---------------------------------------------------------------------------------------------- */

/* One 16(k) x 64(n) tile -> 128 words.  For "warp" w in 0..3 and lane t in 0..31 the output word
 * t*4+w gathers 8 codes: rows (t%4)*2 + {0,1,8,9}, columns w*16 + t/4 and +8, packed in order
 * {0,2,4,6,1,3,5,7}.  K/gptq_marlin/gptq_marlin_repack.cu:138-235, constants K/gptq_marlin/marlin.cuh:45-54. */
static void marlin_tile(const uint8_t* codes, size_t N, size_t k0, size_t n0, uint32_t* out) {
  static const int tc_offsets[4] = {0, 1, 8, 9};
  static const int pack_idx[8] = {0, 2, 4, 6, 1, 3, 5, 7};
  for (int w = 0; w < 4; ++w)
    for (int t = 0; t < 32; ++t) {
      int tc_col = t / 4, tc_row = (t % 4) * 2;
      size_t cur_n = n0 + (size_t)w * 16 + tc_col;
      uint32_t vals[8];
      for (int i = 0; i < 4; ++i) {
        size_t k = k0 + tc_row + tc_offsets[i];
        vals[i] = codes[k * N + cur_n];
        vals[4 + i] = codes[k * N + cur_n + 8];
      }
      uint32_t res = 0;
      for (int i = 0; i < 8; ++i) res |= (vals[pack_idx[i]] & 0xf) << (4 * i);
      out[t * 4 + w] = res;
    }
}

static void marlin_from_codes(const uint8_t* codes, uint32_t* out, size_t K, size_t N) {
  size_t k_tiles = K / 16, n_tiles = N / 64;
  for (size_t kt = 0; kt < k_tiles; ++kt)
    for (size_t nt = 0; nt < n_tiles; ++nt) marlin_tile(codes, N, kt * 16, nt * 64, out + (kt * n_tiles + nt) * 128);
}

/* gptq_marlin_repack without act-order: [K/8, N] int32 -> [K/16, 2N] int32.
 * K/gptq_marlin/gptq_marlin_repack.cu:35-265,297-300. */
KSQO_API int ksqo_marlin_gptq_repack(const uint32_t* qweight, uint32_t* out, size_t K, size_t N) {
  uint8_t* codes = (uint8_t*)malloc(K * N);
  if (!codes) return -1;
  ksqo_gptq_unpack(qweight, codes, K, N);
  marlin_from_codes(codes, out, K, N);
  free(codes);
  return 0;
}

/* awq_marlin_repack: [K, N/8] int32 -> [K/16, 2N] int32.  K/gptq_marlin/awq_marlin_repack.cu:34-206,224-228. */
KSQO_API int ksqo_marlin_awq_repack(const uint32_t* qweight, uint32_t* out, size_t K, size_t N) {
  uint8_t* codes = (uint8_t*)malloc(K * N);
  if (!codes) return -1;
  ksqo_awq_unpack(qweight, codes, K, N);
  marlin_from_codes(codes, out, K, N);
  free(codes);
  return 0;
}

/* MarlinAwqToMarlinZeroPoints: [R, N/8] int32 AWQ-packed zeros -> [R, N/8] int32 Marlin zeros.
 * S/models/quant/marlin_utils.cpp:36-104.  Steps, all on a [R, N] code matrix:
 *   1. MarlinUnpackCols: column 8j+i <- nibble i of word j (plain order)
 *   2. undo AWQ interleave: within each run of 8, index_select by argsort({0,2,4,6,1,3,5,7}) = {0,4,1,5,2,6,3,7}
 *   3. MarlinZeroPoints: within each run of 64, select i + 8*j order (scale_perm), then within each run of 8
 *      select {0,2,4,6,1,3,5,7}, then MarlinPackCols: word j nibble i <- column i-strided: column j + i*(N/8)
 */
KSQO_API int ksqo_marlin_awq_zero_points(const uint32_t* qz, uint32_t* out, size_t R, size_t N) {
  static const int undo[8] = {0, 4, 1, 5, 2, 6, 3, 7};
  static const int inter[8] = {0, 2, 4, 6, 1, 3, 5, 7};
  size_t total = R * N;
  uint8_t* a = (uint8_t*)malloc(total);
  uint8_t* b = (uint8_t*)malloc(total);
  if (!a || !b) {
    free(a);
    free(b);
    return -1;
  }
  size_t NP = N / 8;
  /* 1: q_res[:, i::8] = (packed >> 4i) & 15  -> column i + 8*j... index_put with Slice(i, None, 8) */
  for (size_t r = 0; r < R; ++r)
    for (size_t j = 0; j < NP; ++j) {
      uint32_t w = qz[r * NP + j];
      for (int i = 0; i < 8; ++i) a[r * N + j * 8 + i] = (uint8_t)((w >> (4 * i)) & 0xf);
    }
  /* 2: reshape(-1, 8).index_select(1, undo) */
  for (size_t g = 0; g < total / 8; ++g)
    for (int i = 0; i < 8; ++i) b[g * 8 + i] = a[g * 8 + undo[i]];
  /* 3a: reshape(-1, 64).index_select(1, scale_perm) with scale_perm[i*8+j] = i + 8*j */
  for (size_t g = 0; g < total / 64; ++g)
    for (int i = 0; i < 8; ++i)
      for (int j = 0; j < 8; ++j) a[g * 64 + i * 8 + j] = b[g * 64 + i + 8 * j];
  /* 3b: reshape(-1, 8).index_select(1, interleave) */
  for (size_t g = 0; g < total / 8; ++g)
    for (int i = 0; i < 8; ++i) b[g * 8 + i] = a[g * 8 + inter[i]];
  /* 3c: MarlinPackCols: q_res |= q_w[:, i::8] << 4i  -> word j takes column 8*j + i */
  for (size_t r = 0; r < R; ++r)
    for (size_t j = 0; j < NP; ++j) {
      uint32_t w = 0;
      for (int i = 0; i < 8; ++i) w |= (uint32_t)(b[r * N + j * 8 + i] & 0xf) << (4 * i);
      out[r * NP + j] = w;
    }
  free(a);
  free(b);
  return 0;
}

/* ------------------------------------------------------------------------------------------------
 * W4A16: dequant + fp32 GEMM
 * ---------------------------------------------------------------------------------------------- */

/* w[k,n] = (code[k,n] - zp) * s[k/group, n]; zp = 8 for GPTQ-symmetric (zeros == NULL) or zeros[k/group, n].
 * Scale is widened to fp32 first.  S/layers/layer_test.cpp:451-470 (GetRefGptq), K/machete/machete_wrapper.cu:16-59;
 * AWQ form s*(q-z) from S/models/quant/quant_weight.cpp:735-741. */
KSQO_API void ksqo_w4a16_dequant(const uint8_t* codes, const void* scales, const uint8_t* zeros, float* w, size_t K,
                                 size_t N, size_t group, int dtype) {
#pragma omp parallel for schedule(static)
  for (size_t k = 0; k < K; ++k) {
    size_t g = k / group;
    for (size_t n = 0; n < N; ++n) {
      float s = load_t(scales, g * N + n, dtype);
      float zp = zeros ? (float)zeros[g * N + n] : 8.0f;
      w[k * N + n] = ((float)codes[k * N + n] - zp) * s;
    }
  }
}

/* y[M,N] = x[M,K] * w[K,N], x given in dtype, fp32 accumulate in ascending k, result left in fp32. */
KSQO_API void ksqo_gemm_xw_f32(const void* x, const float* w, float* y, size_t M, size_t N, size_t K, int dtype) {
  float* xf = (float*)malloc(M * K * sizeof(float));
  for (size_t i = 0; i < M * K; ++i) xf[i] = load_t(x, i, dtype);
#pragma omp parallel for schedule(static)
  for (size_t n0 = 0; n0 < N; n0 += 64) {
    size_t n1 = n0 + 64 < N ? n0 + 64 : N;
    for (size_t m = 0; m < M; ++m) {
      float acc[64];
      for (size_t j = 0; j < 64; ++j) acc[j] = 0.f;
      for (size_t k = 0; k < K; ++k) {
        float xv = xf[m * K + k];
        const float* wr = w + k * N + n0;
        for (size_t j = 0; j < n1 - n0; ++j) acc[j] += xv * wr[j];
      }
      for (size_t j = 0; j < n1 - n0; ++j) y[m * N + n0 + j] = acc[j];
    }
  }
  free(xf);
}

/* Same product with a float64 accumulator; used to bound the fp32 oracle's own error in tests. */
KSQO_API void ksqo_gemm_xw_f64(const void* x, const float* w, double* y, size_t M, size_t N, size_t K, int dtype) {
#pragma omp parallel for schedule(static)
  for (size_t n0 = 0; n0 < N; n0 += 64) {
    size_t n1 = n0 + 64 < N ? n0 + 64 : N;
    for (size_t m = 0; m < M; ++m) {
      double acc[64];
      for (size_t j = 0; j < 64; ++j) acc[j] = 0.0;
      for (size_t k = 0; k < K; ++k) {
        double xv = (double)load_t(x, m * K + k, dtype);
        const float* wr = w + k * N + n0;
        for (size_t j = 0; j < n1 - n0; ++j) acc[j] += xv * (double)wr[j];
      }
      for (size_t j = 0; j < n1 - n0; ++j) y[m * N + n0 + j] = acc[j];
    }
  }
}

/* Dequantize-then-GEMM in one call: the CPU baseline the benchmark times. */
KSQO_API int ksqo_w4a16_gemm(const void* x, const uint8_t* codes, const void* scales, const uint8_t* zeros, float* y,
                             size_t M, size_t N, size_t K, size_t group, int dtype) {
  float* w = (float*)malloc(K * N * sizeof(float));
  if (!w) return -1;
  ksqo_w4a16_dequant(codes, scales, zeros, w, K, N, group, dtype);
  ksqo_gemm_xw_f32(x, w, y, M, N, K, dtype);
  free(w);
  return 0;
}

/* ------------------------------------------------------------------------------------------------
 * FP8 per-token-group activation quantizer
 * ---------------------------------------------------------------------------------------------- */

/* K/others/sglang/main/quantization/fp8/per_token_group_quant.cu:105-222:
 *   amax = max(1e-10, max|x|) over the group; s = amax / 448 (IEEE fp32 division);
 *   q = e4m3_rne_satfinite(x / s) (IEEE division); scales [m, k/group] row-major or [k/group, m] column-major.
 * fuse_silu_mul: input is [m, 2k]; x = T(silu(gate) * up) with gate = first half (lines 150-176). */
KSQO_API void ksqo_fp8_group_quant(const void* x, uint8_t* q, float* s, size_t m, size_t k, size_t group,
                                   int column_major, int fuse_silu_mul, int dtype) {
  size_t ng = k / group;
  size_t in_stride = fuse_silu_mul ? 2 * k : k;
#pragma omp parallel for schedule(static)
  for (size_t t = 0; t < m; ++t) {
    float* buf = (float*)malloc(group * sizeof(float));
    for (size_t g = 0; g < ng; ++g) {
      float amax = 1e-10f;
      for (size_t j = 0; j < group; ++j) {
        size_t idx = t * in_stride + g * group + j;
        float v = load_t(x, idx, dtype);
        if (fuse_silu_mul) {
          float u = load_t(x, idx + k, dtype);
          float h = 0.5f * v;
          v = round_t(h * (1.0f + tanhf(h)) * u, dtype);
        }
        buf[j] = v;
        float a = fabsf(v);
        amax = fmaxf(amax, a);
      }
      volatile float scale = amax / 448.0f;
      s[column_major ? g * m + t : t * ng + g] = scale;
      for (size_t j = 0; j < group; ++j) {
        volatile float r = buf[j] / scale;
        q[t * k + g * group + j] = ksqo_f32_to_e4m3(r);
      }
    }
    free(buf);
  }
}

/* ------------------------------------------------------------------------------------------------
 * Per-tensor / per-channel FP8
 * ---------------------------------------------------------------------------------------------- */

/* 3rdparty/LLM_kernels/csrc/utils/nvidia/cuda_fp8_utils.cu:150-256 (scale) and :32-41 (quantize), as called by
 * Fp8E4m3Quantize (S/kernels/nvidia/basic_kernel_wrapper.cpp:1028-1036):
 *   dynamic: scale[c] = max(amax|x[c,:]| / 448, 1/(448*512));  q = e4m3(min(max(x / scale, -448), 448)).
 * Pinned by tests/test_oracle_golden.py against torch's float8_e4m3fn conversion and the reference test's formula
 * (utils_test.cu:48-56, 136-143). */
KSQO_API void ksqo_fp8_channel_quant(const void* x, uint8_t* q, float* scale, size_t channels, size_t size,
                                     int is_static, int dtype) {
  for (size_t c = 0; c < channels; ++c) {
    if (!is_static) {
      float amax = 0.f;
      for (size_t i = 0; i < size; ++i) amax = fmaxf(amax, fabsf(load_t(x, c * size + i, dtype)));
      volatile float sc = amax / 448.0f;
      scale[c] = fmaxf(sc, 1.0f / 448.0f / 512.0f);
    }
    volatile float sc = scale[c];
    for (size_t i = 0; i < size; ++i) {
      volatile float r = load_t(x, c * size + i, dtype) / sc;
      q[c * size + i] = ksqo_f32_to_e4m3(fminf(fmaxf(r, -448.0f), 448.0f));
    }
  }
}

/* out[m,n] = (sum_k a[m,k] * b[n,k]) * a_scale * b_scale: what cuBLASLt computes for Fp8QuantizedMatMul
 * (S/kernels/nvidia/basic_kernel_wrapper.cpp:1042-1052: e4m3 x e4m3, fp32 compute type, scale pointers).
 * The sum is taken in double here, so the result is the exact value up to the final rounding. */
KSQO_API void ksqo_fp8_tensor_gemm(const uint8_t* a, float a_scale, const uint8_t* b, float b_scale, float* out, size_t m,
                                   size_t n, size_t k) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = ksqo_e4m3_to_f32((uint8_t)i);
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i)
    for (size_t j = 0; j < n; ++j) {
      double acc = 0.0;
      for (size_t kk = 0; kk < k; ++kk) acc += (double)lut[a[i * k + kk]] * (double)lut[b[j * k + kk]];
      out[i * n + j] = (float)(acc * (double)a_scale * (double)b_scale);
    }
}

/* ------------------------------------------------------------------------------------------------
 * Blockwise FP8 GEMM
 * ---------------------------------------------------------------------------------------------- */

/* out[m,n] = sum_kb ( sum_{k in kb} a[m,k] * b[n,k] ) * a_s[m,kb] * b_s[n/128, kb]
 * a [m,k] e4m3 row-major, b [n,k] e4m3 row-major, a_s column-major [k/128, m] (or row-major [m, k/128] when
 * a_s_column_major == 0), b_s [ceil(n/128), k/128].  fp32 partial per 128-k block, fp32 outer accumulator.
 * K/blockwise_gemm/blockwise_gemm_test.cu:138-177; scale layouts S/layers/nvidia/blockwise_matmul_layer.cpp:262-272. */
KSQO_API void ksqo_fp8_blockwise_gemm(const uint8_t* a, const float* a_s, const uint8_t* b, const float* b_s,
                                      float* out, size_t m, size_t n, size_t k, int a_s_column_major) {
  const size_t B = 128;
  size_t kt = (k + B - 1) / B;
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = ksqo_e4m3_to_f32((uint8_t)i);
  float* af = (float*)malloc(m * k * sizeof(float));
  for (size_t i = 0; i < m * k; ++i) af[i] = lut[a[i]];
#pragma omp parallel for schedule(static)
  for (size_t col = 0; col < n; ++col) {
    float* bf = (float*)malloc(k * sizeof(float));
    for (size_t l = 0; l < k; ++l) bf[l] = lut[b[col * k + l]];
    for (size_t row = 0; row < m; ++row) {
      float acc = 0.f;
      for (size_t kb = 0; kb < kt; ++kb) {
        size_t k1 = (kb + 1) * B < k ? (kb + 1) * B : k;
        float sum = 0.f;
        for (size_t l = kb * B; l < k1; ++l) sum += af[row * k + l] * bf[l];
        float as = a_s_column_major ? a_s[kb * m + row] : a_s[row * kt + kb];
        acc += sum * (as * b_s[(col / B) * kt + kb]);
      }
      out[row * n + col] = acc;
    }
    free(bf);
  }
  free(af);
}

/* Weight-side 128x128 block quantizer used to build synthetic fp8 weights: s = amax/448 per block,
 * q = e4m3(w / s).  S/kernels/nvidia/basic_kernel_wrapper.cpp:1147-1193 (ScaledQuantizeFp8E4m3). */
KSQO_API void ksqo_fp8_block_quant_weight(const float* w, uint8_t* q, float* s, size_t n, size_t k) {
  const size_t B = 128;
  size_t nb = (n + B - 1) / B, kb = (k + B - 1) / B;
#pragma omp parallel for schedule(static)
  for (size_t bi = 0; bi < nb; ++bi)
    for (size_t bj = 0; bj < kb; ++bj) {
      float amax = 0.f;
      size_t r1 = (bi + 1) * B < n ? (bi + 1) * B : n, c1 = (bj + 1) * B < k ? (bj + 1) * B : k;
      for (size_t r = bi * B; r < r1; ++r)
        for (size_t c = bj * B; c < c1; ++c) amax = fmaxf(amax, fabsf(w[r * k + c]));
      float sc = amax > 0.f ? amax / 448.0f : 1.0f;
      s[bi * kb + bj] = sc;
      for (size_t r = bi * B; r < r1; ++r)
        for (size_t c = bj * B; c < c1; ++c) q[r * k + c] = ksqo_f32_to_e4m3(w[r * k + c] / sc);
    }
}

/* ------------------------------------------------------------------------------------------------
 * MoE: align, grouped W4A16 GEMM, silu*mul, weighted sum
 * ---------------------------------------------------------------------------------------------- */

/* Counting sort of topk_ids by expert, each expert's segment padded to block_size with the value numel.
 * Stable (ascending flat index inside an expert).  sorted_ids must hold numel + E*(block_size-1) entries and is
 * fully pre-filled with numel; expert_ids holds one entry per block.  ids >= E are skipped.
 * S/kernels/nvidia/fused_moe_gptq_awq_test.cpp:54-83 (MoeAlignBlockCpu), K/moe_utils/moe_utils.cu:92-169. */
KSQO_API int ksqo_moe_align(const int32_t* topk_ids, size_t numel, int E, int block_size, int32_t* sorted_ids,
                            int32_t* expert_ids, int32_t* num_post_pad) {
  size_t cap = numel + (size_t)E * (size_t)(block_size - 1);
  int32_t* cumsum = (int32_t*)calloc((size_t)E + 1, sizeof(int32_t));
  int32_t* cnt = (int32_t*)calloc((size_t)E + 1, sizeof(int32_t));
  if (!cumsum || !cnt) return -1;
  for (size_t i = 0; i < cap; ++i) sorted_ids[i] = (int32_t)numel;
  for (size_t i = 0; i < numel; ++i) {
    int e = topk_ids[i];
    if (e < 0 || e >= E) continue;
    cnt[e] += 1;
  }
  for (int e = 0; e < E; ++e) {
    cumsum[e + 1] = cumsum[e] + (cnt[e] + block_size - 1) / block_size;
    cnt[e] = 0;
    for (int j = cumsum[e]; j < cumsum[e + 1]; ++j) expert_ids[j] = e;
  }
  num_post_pad[0] = cumsum[E] * block_size;
  for (size_t i = 0; i < numel; ++i) {
    int e = topk_ids[i];
    if (e < 0 || e >= E) continue;
    sorted_ids[(size_t)cumsum[e] * block_size + cnt[e]] = (int32_t)i;
    cnt[e] += 1;
  }
  free(cumsum);
  free(cnt);
  return 0;
}

/* Grouped W4A16 GEMM for one MoE stage, dense restatement (no sorting needed on the CPU):
 *   out[t*top_k_out + j, :] = ( x[row(t,j), :] . dequant(W[e]) ) * (mul_routed ? topk_w[t*top_k_out+j] : 1)
 * with e = topk_ids[...] and row(t,j) = (t*top_k_out + j) / top_k_div, which is the reference's
 * "offs_token // top_k" (K/moe/fused_moe_kernel_gptq_awq/fused_moe_kernel_gptq_awq.py:172-177,243-269):
 * stage 1 reads token t for every slot (top_k_div = topk), stage 2 reads slot rows directly (top_k_div = 1).
 * W [E, N, K/2] u8 low nibble = even k, w = (code - 8) * s, scales [E, N, K/group] in dtype
 * (S/kernels/nvidia/fused_moe_gptq_awq_test.cpp:119-124).  The accumulator is rounded to dtype after the routed
 * weight is applied in fp32, as the store `accumulator.to(compute_type)` does. */
KSQO_API void ksqo_moe_w4a16_gemm(const void* x, const uint8_t* w, const void* scales, const int32_t* topk_ids,
                                  const float* topk_w, float* out, size_t num_slots, int top_k_div, size_t N,
                                  size_t K, size_t group, int mul_routed, int dtype) {
  size_t ng = K / group;
#pragma omp parallel for schedule(dynamic, 1)
  for (size_t slot = 0; slot < num_slots; ++slot) {
    int e = topk_ids[slot];
    size_t row = slot / (size_t)top_k_div;
    float* xf = (float*)malloc(K * sizeof(float));
    for (size_t kk = 0; kk < K; ++kk) xf[kk] = load_t(x, row * K + kk, dtype);
    for (size_t n = 0; n < N; ++n) {
      const uint8_t* wr = w + ((size_t)e * N + n) * (K / 2);
      float acc = 0.f;
      for (size_t g = 0; g < ng; ++g) {
        float s = load_t(scales, ((size_t)e * N + n) * ng + g, dtype);
        float part = 0.f;
        for (size_t kk = g * group; kk < (g + 1) * group; kk += 2) {
          uint8_t b = wr[kk / 2];
          part += xf[kk] * (float)((int)(b & 0xf) - 8);
          part += xf[kk + 1] * (float)((int)(b >> 4) - 8);
        }
        acc += part * s;
      }
      if (mul_routed) acc *= topk_w[slot];
      out[slot * N + n] = acc;
    }
    free(xf);
  }
}

/* Router: fp32 softmax over the experts, top_k by repeated arg-max (lowest id wins ties), weight = prob * scaling,
 * or prob / sum(top_k probs) * scaling when norm is set.  K/grouped_topk/grouped_topk.cu:678-733
 * (BasicSoftmaxTopkKernel); the renormalisation is the norm_topk_prob option of the layer above it. */
KSQO_API void ksqo_moe_topk_softmax(const void* gating, float* topk_w, int32_t* topk_ids, size_t tokens, size_t E,
                                    size_t top_k, int norm, float scaling, int dtype) {
#pragma omp parallel for schedule(static)
  for (size_t t = 0; t < tokens; ++t) {
    float* sc = (float*)malloc(E * sizeof(float));
    float mx = load_t(gating, t * E, dtype);
    for (size_t e = 0; e < E; ++e) {
      sc[e] = load_t(gating, t * E + e, dtype);
      mx = fmaxf(mx, sc[e]);
    }
    float sum = 0.f;
    for (size_t e = 0; e < E; ++e) {
      sc[e] = expf(sc[e] - mx);
      sum += sc[e];
    }
    float picked = 0.f;
    for (size_t r = 0; r < top_k; ++r) {
      size_t best = 0;
      float bv = -2.f;
      for (size_t e = 0; e < E; ++e)
        if (sc[e] > bv) {
          bv = sc[e];
          best = e;
        }
      sc[best] = -1.f;
      topk_ids[t * top_k + r] = (int32_t)best;
      topk_w[t * top_k + r] = bv / sum;
      picked += bv / sum;
    }
    for (size_t r = 0; r < top_k; ++r)
      topk_w[t * top_k + r] = (norm ? topk_w[t * top_k + r] / picked : topk_w[t * top_k + r]) * scaling;
    free(sc);
  }
}

/* Grouped router.  Follows the reference's CPU restatement of DeepSeek-V3 routing
 * (3rdparty/LLM_kernels/tests/references/deepseek_v3_grouped_topk.h:139-236: sigmoid, + bias, group rank = sum of the
 * two largest, top groups, top_k over the kept groups, weights from the unbiased scores, / sum * scaling) and the
 * tensor-op form of S/kernels/nvidia/moe_kernel_wrapper.cpp:286-347 for the other options (softmax scoring, no
 * bias -> group rank = largest, renormalize off, experts outside the kept groups excluded outright).
 * Picks are by repeated arg-max, the lower index winning ties.
 * Pinned by tests/test_oracle_golden.py against the published DeepSeek-V3 formula written with torch tensor ops and
 * against that reference header itself, compiled from the reference tree into oracle/_ref (ref_grouped_topk.cpp). */
KSQO_API void ksqo_moe_grouped_topk(const void* gating, const float* bias, float* topk_w, int32_t* topk_ids,
                                    size_t tokens, size_t E, size_t top_k, size_t groups, size_t topk_group,
                                    int sigmoid, int renorm, float scaling, int dtype) {
  const size_t per = E / groups;
#pragma omp parallel for schedule(static)
  for (size_t t = 0; t < tokens; ++t) {
    float* score = (float*)malloc(E * sizeof(float));
    float* choose = (float*)malloc(E * sizeof(float));
    float* rank = (float*)malloc(groups * sizeof(float));
    char* kept = (char*)calloc(groups, 1);
    char* taken = (char*)calloc(E, 1);
    if (sigmoid) {
      for (size_t e = 0; e < E; ++e) score[e] = 1.0f / (1.0f + expf(-load_t(gating, t * E + e, dtype)));
    } else {
      float mx = load_t(gating, t * E, dtype), sum = 0.f;
      for (size_t e = 0; e < E; ++e) mx = fmaxf(mx, load_t(gating, t * E + e, dtype));
      for (size_t e = 0; e < E; ++e) {
        score[e] = expf(load_t(gating, t * E + e, dtype) - mx);
        sum += score[e];
      }
      for (size_t e = 0; e < E; ++e) score[e] = score[e] / sum;
    }
    for (size_t e = 0; e < E; ++e) choose[e] = score[e] + (bias ? bias[e] : 0.f);
    for (size_t g = 0; g < groups; ++g) {
      float m1 = -INFINITY, m2 = -INFINITY;
      for (size_t i = 0; i < per; ++i) {
        const float c = choose[g * per + i];
        if (c > m1) {
          m2 = m1;
          m1 = c;
        } else if (c > m2) {
          m2 = c;
        }
      }
      rank[g] = bias ? m1 + m2 : m1;
    }
    for (size_t r = 0; r < topk_group; ++r) {
      size_t best = groups;
      for (size_t g = 0; g < groups; ++g)
        if (!kept[g] && (best == groups || rank[g] > rank[best])) best = g;
      kept[best] = 1;
    }
    float picked = 0.f;
    for (size_t r = 0; r < top_k; ++r) {
      size_t best = E;
      for (size_t e = 0; e < E; ++e)
        if (kept[e / per] && !taken[e] && (best == E || choose[e] > choose[best])) best = e;
      topk_ids[t * top_k + r] = (int32_t)best;
      topk_w[t * top_k + r] = score[best];
      picked += score[best];
      taken[best] = 1;
    }
    for (size_t r = 0; r < top_k; ++r)
      topk_w[t * top_k + r] = (renorm ? topk_w[t * top_k + r] / picked : topk_w[t * top_k + r]) * scaling;
    free(score);
    free(choose);
    free(rank);
    free(kept);
    free(taken);
  }
}

/* out[r, i] = T( silu(a) * b ) with a = x[r, i], b = x[r, inter + i], math in fp32: a / (1 + expf(-a)) * b.
 * K/moe_utils/moe_utils.cu:597-606. */
KSQO_API void ksqo_silu_mul(const void* x, void* out, size_t rows, size_t inter, int dtype) {
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; ++r)
    for (size_t i = 0; i < inter; ++i) {
      float a = load_t(x, r * 2 * inter + i, dtype);
      float b = load_t(x, r * 2 * inter + inter + i, dtype);
      store_t(out, r * inter + i, a / (1.0f + expf(-a)) * b, dtype);
    }
}

/* out[t, :] = sum_j in[t, j, :], accumulated IN dtype precision, j ascending.  K/moe_utils/moe_utils.cu:549-562. */
KSQO_API void ksqo_moe_sum(const void* in, void* out, size_t tokens, size_t topk, size_t d, int dtype) {
#pragma omp parallel for schedule(static)
  for (size_t t = 0; t < tokens; ++t)
    for (size_t i = 0; i < d; ++i) {
      float acc = 0.f;
      for (size_t j = 0; j < topk; ++j) acc = round_t(acc + load_t(in, (t * topk + j) * d + i, dtype), dtype);
      store_t(out, t * d + i, acc, dtype);
    }
}

/* ------------------------------------------------------------------------------------------------
 * W4A8 (FinegrainedMixedDtypeGemmLayer)
 * ---------------------------------------------------------------------------------------------- */

/* [K, N/2] packed bytes -> [K, N] int8: low nibble = even column, both sign-extended
 * (finegrained_mixed_dtype_gemm_thop_test.cu:53-80). */
KSQO_API void ksqo_w4a8_unpack_int4(const int8_t* w, int8_t* out, size_t K, size_t N) {
  for (size_t i = 0; i < K * (N / 2); ++i) {
    const int8_t b = w[i];
    out[2 * i] = (int8_t)((int8_t)(b << 4) >> 4);
    out[2 * i + 1] = (int8_t)(b >> 4);
  }
}

/* q[i] = e4m3(float(x[i]) / scale), scale = scale[0] (mode 0), scale[i % k] (mode 1) or scale[i / k] (mode 3):
 * scaleMatrix<PER_TENSOR | PER_CHANNEL | PER_TOKEN, true> (K/others/tensorrt-llm/dev/common/cudaFp8Utils.cu:33-52);
 * the conversion saturates to +-448 (__nv_fp8_e4m3). */
KSQO_API void ksqo_w4a8_static_quant(const void* x, const float* scale, uint8_t* q, size_t m, size_t k, int mode,
                                     int dtype) {
  for (size_t i = 0; i < m * k; ++i) {
    volatile float sc = mode == 1 ? scale[i % k] : (mode == 3 ? scale[i / k] : scale[0]);
    volatile float r = load_t(x, i, dtype) / sc;
    q[i] = ksqo_f32_to_e4m3(fminf(fmaxf(r, -448.0f), 448.0f));
  }
}

/* xsum[m, g] = sum of the 128 decoded e4m3 values of group g (in double, rounded once). */
KSQO_API void ksqo_w4a8_group_sums_g(const uint8_t* q, float* xsum, size_t m, size_t k, size_t group) {
  for (size_t i = 0; i < m; ++i)
    for (size_t g = 0; g < k / group; ++g) {
      double acc = 0.0;
      for (size_t j = 0; j < group; ++j) acc += (double)ksqo_e4m3_to_f32(q[i * k + g * group + j]);
      xsum[i * (k / group) + g] = (float)acc;
    }
}
KSQO_API void ksqo_w4a8_group_sums(const uint8_t* q, float* xsum, size_t m, size_t k) {
  ksqo_w4a8_group_sums_g(q, xsum, m, k, 128);
}

/* out[m,n] = alpha * sum_k a[m,k] * (w[k,n] * scale[k/group, n]): the reference test's formula
 * (finegrained_mixed_dtype_gemm_thop_test.cu:186-206: unpack, multiply by the repeated scales, matmul of the
 * alpha-scaled activations), taken in double here so that the result is the exact value up to the last rounding.
 * a [m,k] e4m3, w [k,n/2] packed int4 as above, scales fp16 [k/group, n]. */
KSQO_API void ksqo_w4a8_gemm(const uint8_t* a, const int8_t* w, const uint16_t* scales, float alpha, float* out,
                             size_t m, size_t n, size_t k, size_t group) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = ksqo_e4m3_to_f32((uint8_t)i);
  double* wd = (double*)malloc(sizeof(double) * k * n);
  for (size_t kk = 0; kk < k; ++kk)
    for (size_t j = 0; j < n; ++j) {
      const int8_t b = w[kk * (n / 2) + j / 2];
      const int v = (j & 1) ? (b >> 4) : ((int8_t)(b << 4) >> 4);
      wd[kk * n + j] = (double)v * (double)ksqo_f16_to_f32(scales[(kk / group) * n + j]);
    }
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < m; ++i) {
    double* acc = (double*)calloc(n, sizeof(double));
    for (size_t kk = 0; kk < k; ++kk) {
      const double av = (double)lut[a[i * k + kk]];
      if (av == 0.0) continue;
      for (size_t j = 0; j < n; ++j) acc[j] += av * wd[kk * n + j];
    }
    for (size_t j = 0; j < n; ++j) out[i * n + j] = (float)(acc[j] * (double)alpha);
    free(acc);
  }
  free(wd);
}
