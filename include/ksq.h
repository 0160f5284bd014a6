/*
 * ksq.h - C-ABI of libksq_hip.so, the MI355X (gfx950) quantized-GEMM kernel library that sits under
 * KsanaLLM's matmul / MoE layer classes.
 *
 * Conventions
 *   - plain pointers and sizes only; every device pointer is caller-owned HBM;
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream);
 *   - every function that launches work returns an int status (KSQ_OK == 0), never allocates device memory,
 *     never synchronizes; ksq_last_error_string() explains the last non-zero status of the calling thread;
 *   - `dtype` is the activation/output/scale type T of the reference's templates (KSQ_F16 or KSQ_BF16);
 *   - 16-byte alignment is required of every device pointer.
 *
 * Citations name the reference interface each entry point replaces:
 *   S/ = src/ksana_llm/      K/ = 3rdparty/LLM_kernels/csrc/kernels/nvidia/
 */
#ifndef KSQ_H_
#define KSQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KSQ_VERSION 1

/* status codes */
enum {
  KSQ_OK = 0,
  KSQ_ERR_INVALID_ARGUMENT = 1, /* null pointer, misaligned pointer, zero / non-conforming size */
  KSQ_ERR_UNSUPPORTED = 2,      /* valid request the library has no kernel for (dtype, group size ...) */
  KSQ_ERR_WORKSPACE = 3,        /* workspace smaller than ksq_*_workspace_size() reported */
  KSQ_ERR_LAUNCH = 4            /* hipGetLastError() after the launch was not hipSuccess */
};

/* element type tags */
enum { KSQ_F16 = 0, KSQ_BF16 = 1, KSQ_F32 = 2 };

/* checkpoint-side int4 weight layouts accepted by the repack (what the loader holds after slicing) */
enum {
  KSQ_SRC_GPTQ = 0,    /* [E][K/8, N] int32, nibble i of a word = row 8*(k/8)+i     (S/models/quant/cutlass_utils.cpp:41-50) */
  KSQ_SRC_AWQ = 1,     /* [E][K, N/8] int32, AWQ column order {0,2,4,6,1,3,5,7}     (S/models/quant/cutlass_utils.cpp:12-38) */
  KSQ_SRC_MOE_NK = 2,  /* [E, N, K/2] uint8, low nibble = even k                    (S/models/quant/quant_weight.cpp:182-319) */
  KSQ_SRC_INT4X2_KN = 3 /* [E][K, N/2] int8, two signed nibbles (code-8), low = even n (S/models/quant/cutlass_utils.cpp:53-59) */
};

/* scale / zero-point source layouts */
enum {
  KSQ_SCALE_GN = 0, /* [E][K/group, N]   dense GPTQ / AWQ checkpoints */
  KSQ_SCALE_NG = 1  /* [E, N, K/group]   MoE expert stacks (S/models/quant/quant_weight.cpp:182-319) */
};
enum {
  KSQ_ZERO_AWQ_PACKED = 0, /* [K/group, N/8] int32 in AWQ column order (qzeros as stored in the checkpoint) */
  KSQ_ZERO_U8_GN = 1       /* [K/group, N] uint8 codes 0..15 */
};

int ksq_version(void);

/* Replaces the cudaGetErrorString / KLLM_KERNEL_CHECK text paths.  Thread-local, never NULL. */
const char* ksq_last_error_string(void);

/* ------------------------------------------------------------------------------------------------------------------
 * Load-time repack: checkpoint layout <-> CDNA4 tile layout.
 *
 * The packed weight is a sequence of 1 KiB tiles, tile (e, n/16, k/128) at ((e*N/16 + n/16)*(K/128) + k/128).
 * Inside a tile, wavefront lane l = 16*((k%32)/8) + n%16 owns 16 bytes; dword d = (k%128)/32 of those bytes holds
 * the eight codes k%8 = {0,2,4,6,1,3,5,7} from nibble 0 upward, so `(w >> 4i) & 0x000F000F` is the MFMA operand
 * pair (k=2i, k=2i+1).  Scales are [e][n/16][K/group][16] in T, zero points the same shape in uint8.
 * K must be a multiple of 128, N of 16, group one of 32/64/128.
 *
 * Replaces fast_preprocess_weights_for_mixed_gemm (K/asymmetric_gemm/cutlass_preprocessors_fast.cu:370),
 * gptq_marlin_repack / awq_marlin_repack (K/gptq_marlin/gptq_marlin_repack.cu:276-295, awq_marlin_repack.cu:208-222),
 * machete_prepack_weight (K/machete/machete_wrapper.h:38-109), permute_scales (K/gptq_marlin/gptq_marlin.cu:641-682)
 * and the AWQ zero-point conversions (S/models/quant/quant_weight.cpp:716-753, S/models/quant/marlin_utils.cpp:36-104).
 * ------------------------------------------------------------------------------------------------------------------ */
size_t ksq_w4a16_packed_weight_bytes(size_t E, size_t K, size_t N);
size_t ksq_w4a16_packed_scales_bytes(size_t E, size_t K, size_t N, size_t group, int dtype);
size_t ksq_w4a16_packed_zeros_bytes(size_t E, size_t K, size_t N, size_t group);

int ksq_w4a16_repack(const void* src, int src_layout, void* dst_packed, size_t E, size_t K, size_t N, void* stream);
/* exact inverse of ksq_w4a16_repack for every src_layout */
int ksq_w4a16_unpack(const void* packed, int dst_layout, void* dst, size_t E, size_t K, size_t N, void* stream);

/* GPTQ act-order (desc_act) checkpoints: g_idx[k] names the quantization group of input channel k.  With
 * perm = stable argsort(g_idx) (host side, once), packed row j takes checkpoint row perm[j]; every group's rows are
 * then adjacent, scales / zeros apply as for a checkpoint without act-order, and the GEMM reads x[:, perm]
 * (ksq_permute_columns) - together y = x . W exactly as with g_idx.  src [K/8, N] int32 (KSQ_SRC_GPTQ), perm int32 [K].
 * Replaces gptq_marlin_repack with has_perm (K/gptq_marlin/gptq_marlin_repack.cu:276-295), MarlinSortGIdx
 * (S/models/quant/marlin_utils.cpp:106-122) and the activation permutation inside gptq_marlin_gemm. */
int ksq_w4a16_repack_act_order(const void* src_gptq, const void* perm, void* dst_packed, size_t K, size_t N, void* stream);
/* out[r, j] = x[r, perm[j]], x and out [m, k] T, perm int32 [k]; out must not alias x. */
int ksq_permute_columns(const void* x, const void* perm, void* out, size_t m, size_t k, int dtype, void* stream);

/* Act-order GPTQ weight of which this GPU holds a K range only (row-parallel projection under tensor parallelism,
 * is_k_full = false: S/layers/nvidia/marlin_matmul_layer.cpp:66-96).  The rows of the range belong to arbitrary groups of
 * the whole checkpoint, so after sorting by group the runs of equal group have arbitrary lengths; the loader pads every
 * run to a multiple of 32 rows and the GEMM runs with group size 32 on a scale table with one row per 32 packed rows.
 * ksq_w4a16_repack_rows: packed row j (of K_dst, a multiple of 128) takes checkpoint row rows[j] of src [K_src/8, N];
 *   an index outside [0, K_src) marks a padding row, which takes code 8 (contributes nothing under the symmetric zero point).
 * ksq_gather_columns: out[r, j] = x[r, idx[j]], x [m, k_in], out [m, k_out], 0 where idx[j] is outside [0, k_in).
 * Replaces the g_idx / perm / is_k_full arguments of gptq_marlin_gemm (K/gptq_marlin/gptq_marlin.cu:568-607). */
int ksq_w4a16_repack_rows(const void* src_gptq, const void* rows, void* dst_packed, size_t K_src, size_t K_dst, size_t N,
                          void* stream);
int ksq_gather_columns(const void* x, const void* idx, void* out, size_t m, size_t k_in, size_t k_out, int dtype, void* stream);

/* The same for expert stacks: out[s, j] = x[s / top_k, perm[topk_ids[s], j]] for the numel = tokens * top_k slots
 * (top_k = 1: x holds one row per slot already, as in front of the second MoE GEMM); perm int32 [E, k], out [numel, k]
 * T, read by the grouped GEMM with top_k = 1.  Ids outside [0, E) take expert 0's permutation; the grouped GEMM never
 * reads those rows.  Replaces the perm / sorted-g_idx arguments of fused_marlin_moe
 * (S/layers/nvidia/marlin_moe_layer.cpp:71-93). */
int ksq_moe_permute_columns(const void* x, const void* perm, const void* topk_ids, void* out, size_t numel, size_t k,
                            size_t top_k, size_t E, int dtype, void* stream);

int ksq_w4a16_repack_scales(const void* src, int src_layout, void* dst_packed, size_t E, size_t K, size_t N,
                            size_t group, int dtype, void* stream);
int ksq_w4a16_unpack_scales(const void* packed, int dst_layout, void* dst, size_t E, size_t K, size_t N, size_t group,
                            int dtype, void* stream);
int ksq_w4a16_repack_zeros(const void* src, int src_layout, void* dst_packed, size_t K, size_t N, size_t group,
                           void* stream);
int ksq_w4a16_unpack_zeros(const void* packed, int dst_layout, void* dst, size_t K, size_t N, size_t group,
                           void* stream);

/* FP8 (e4m3) weights: checkpoint layout [E, N, K] row-major <-> 2 KiB MFMA fragments of 16 rows x 128 k.  Fragment
 * (e, n/16, k/128) lies at ((e*N/16 + n/16)*(K/128) + k/128) * 2048; inside, half h (0/1), then wavefront lane
 * l = 16*((k%128)/32) + n%16, then the 16 bytes k%32 in [16h, 16h+16): one 1 KiB load per half is the MFMA operand of
 * v_mfma_f32_16x16x128_f8f6f4, contiguous over the wavefront.  Same size as the source; the scales keep their layout.
 * Every FP8 GEMM below takes its weights in this layout.  N % 16 == 0, K % 128 == 0; exact inverse provided.
 * The reference's FP8 kernels read the checkpoint layout directly (cuBLASLt / DeepGEMM / CUTLASS); this is the FP8
 * counterpart of the int4 repack above and belongs in the loader at the same place
 * (S/models/quant/quant_weight.cpp:817-861, where ConvertFp8E4m3Tensor and the block-scale binding run). */
int ksq_fp8_repack_weight(const void* src, void* dst_packed, size_t E, size_t N, size_t K, void* stream);
int ksq_fp8_unpack_weight(const void* packed, void* dst, size_t E, size_t N, size_t K, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * W4A16 group-wise GEMM: y[m,n] = x[m,k] . ((code - zp) * scale), zp = 8 when zeros_packed == NULL (GPTQ symmetric),
 * else the per-(group,n) zero point (AWQ).  x, y row-major T; weights / scales / zeros in the packed layout above.
 * The kernel variant (decode split-K vs MFMA tile, tile sizes) is chosen internally by ksq_select_tile.
 *
 * Replaces InvokeFpAIntBGroupCudaGemm / InvokeFpAIntBGroupCutlassGemm / InvokeMarlinGemm / InvokeMacheteGemm
 * (S/kernels/nvidia/basic_kernel_wrapper.h:32-115) and their workspace probes
 * (GetFpAIntBGroupCutlassGemmWorkspaceSize, GetMarlinWorkspace K/gptq_marlin/gptq_marlin.cu:610-638).
 * ------------------------------------------------------------------------------------------------------------------ */
size_t ksq_w4a16_workspace_size(size_t max_m, size_t n, size_t k, size_t group, int dtype);
int ksq_w4a16_gemm(void* y, const void* x, const void* w_packed, const void* scales_packed, const void* zeros_packed,
                   void* workspace, size_t workspace_bytes, size_t m, size_t n, size_t k, size_t group, int dtype,
                   void* stream);

/* The same call - same kernels, same plan, same workspace - with the fp32 sums stored as they are: y is [m, n] float
 * (16-byte aligned) and nothing is rounded to T.  For verification: what separates a result from the fp32-accumulated
 * dequantize-then-GEMM reference before the output type's own rounding is added.  The reference keeps the same notion
 * in Marlin's fp32 reduce buffer (c_tmp, K/gptq_marlin/gptq_marlin.cu:610-638), without an entry point for it. */
int ksq_w4a16_gemm_f32(float* y, const void* x, const void* w_packed, const void* scales_packed, const void* zeros_packed,
                       void* workspace, size_t workspace_bytes, size_t m, size_t n, size_t k, size_t group, int dtype,
                       void* stream);

/* The same GEMM without a workspace argument, for callers that cannot allocate or hold device memory of their own at
 * the call site: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  The fp32 partial sums of launches that cut K go through a buffer of
 * KSQ_W4A16_STATIC_WORKSPACE_BYTES that is part of the library's code object (each GPU the library runs on holds it
 * until the process ends); a call whose plan needs more returns KSQ_ERR_WORKSPACE and leaves y untouched - use
 * ksq_w4a16_gemm with a workspace then.  The call allocates nothing and frees nothing.  All calls on one GPU share the
 * buffer: two of them that overlap in time (different streams) race on it; calls on one stream do not.
 * The first call on a device also looks up the buffer's address there and sets the large-LDS attribute of the kernels
 * it launches: make one call per device and kernel variant outside graph capture before capturing any. */
#define KSQ_W4A16_STATIC_WORKSPACE_BYTES (32u << 20)
size_t ksq_w4a16_static_workspace_bytes(void);
int ksq_w4a16_gemm_static(void* y, const void* x, const void* w_packed, const void* scales_packed,
                          const void* zeros_packed, size_t m, size_t n, size_t k, size_t group, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * FP8 (OCP e4m3) per-token, per-`group`-channel activation quantizer.
 *   amax = max(1e-10, max|x|); s = amax / 448; q = e4m3_rne_satfinite(x / s)   (IEEE fp32 divisions)
 * x [m, k] T (or [m, 2k] when fuse_silu_mul: x = T(silu(x[:, :k]) * x[:, k:])), q [m, k] bytes,
 * s fp32 [m, k/group] or, when column_major, [k/group, m].
 * dtype KSQ_F16, KSQ_BF16 or KSQ_F32 (x float, no rounding to T in the fused form): the reference instantiates all three
 * (basic_kernel_wrapper.cpp:1237-1239).
 * Replaces InvokePerTokenGroupQuantFp8E4m3 (S/kernels/nvidia/basic_kernel_wrapper.cpp:1222-1232;
 * K/others/sglang/main/quantization/fp8/per_token_group_quant.cu:275-329).
 * ------------------------------------------------------------------------------------------------------------------ */
int ksq_fp8_group_quant(const void* x, void* q, void* s, size_t m, size_t k, size_t group, int column_major,
                        int fuse_silu_mul, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Blockwise FP8 GEMM: out[m,n] = sum_kb (a_q[m,kb] . b[n,kb]) * a_s[kb,m] * b_s[n/128,kb], fp32 accumulate.
 * a_q [m,k] e4m3 row-major, a_s fp32 column-major [k/128, m], b [n,k] e4m3 in the packed fragment layout (ksq_fp8_repack_weight),
 * b_s fp32 [ceil(n/128), k/128], out [m,n] in out_dtype (KSQ_F16, KSQ_BF16, or KSQ_F32 for fp32 activations: the sums
 * as they are, InvokeBlockGemm<float>, basic_kernel_wrapper.cpp:1096).  k must be a multiple of 128, n of 16.
 * Replaces InvokeBlockGemm / InvokeGetBlockGemmWorkspaceSize (K/blockwise_gemm/blockwise_gemm.cu:17-33) and
 * DeepGEMMWrapper::Gemm / GemmSwapAB (K/gemm/deepgemm/deepgemm_wrapper.cu:33-103).
 * ------------------------------------------------------------------------------------------------------------------ */
size_t ksq_fp8_blockwise_workspace_size(size_t max_m, size_t n, size_t k);
int ksq_fp8_blockwise_gemm(const void* a_q, const void* a_s, const void* b, const void* b_s, void* out, size_t m,
                           size_t n, size_t k, int out_dtype, void* workspace, size_t workspace_bytes, void* stream);
/* The same call with the fp32 sums stored as they are (out [m, n] float, 16-byte aligned): for verification, as
 * ksq_w4a16_gemm_f32.  The reference's own check of this GEMM compares against a host loop that keeps fp32 throughout
 * (K/blockwise_gemm/blockwise_gemm_test.cu:138-177). */
int ksq_fp8_blockwise_gemm_f32(const void* a_q, const void* a_s, const void* b, const void* b_s, float* out, size_t m,
                               size_t n, size_t k, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Per-tensor / per-channel FP8: x [channels, size] T -> q e4m3 with one fp32 scale per channel (channels = 1: per tensor).
 *   dynamic (is_static = 0): scale[c] = max(amax|x[c,:]| / 448, 1 / (448 * 512)) is computed and written first
 *   static  (is_static = 1): scale[c] is read
 *   q = e4m3(clamp(x / scale, -448, 448)), IEEE division, round to nearest even.
 * dtype KSQ_F16, KSQ_BF16 or KSQ_F32 (x float).
 * Replaces Fp8E4m3Quantize (S/kernels/nvidia/basic_kernel_wrapper.cpp:1028-1036) = InvokeComputeFP8QuantizeScale +
 * InvokeQuantizeMatrix (3rdparty/LLM_kernels/csrc/utils/nvidia/cuda_fp8_utils.cu:32-266).
 * ------------------------------------------------------------------------------------------------------------------ */
int ksq_fp8_channel_quant(const void* x, void* q, void* scale, size_t channels, size_t size, int is_static, int dtype,
                          void* stream);

/* Per-tensor-scaled FP8 GEMM: out[m,n] = T((sum_k a_q[m,k] . b[n,k]) * a_scale[0] * b_scale[0]), fp32 accumulation.
 * a_q [m,k] e4m3 row-major, b [n,k] e4m3 packed by ksq_fp8_repack_weight; a_scale, b_scale: one fp32 each in device
 * memory.  k % 128 == 0, n % 16 == 0.  out_dtype KSQ_F16, KSQ_BF16 or KSQ_F32 (fp32 activations: the scaled sums as
 * they are).
 * The workspace (256-byte aligned) holds the scales spread into the blockwise layouts and the split-K partials of
 * the blockwise kernels, which do the work.
 * Replaces Fp8QuantizedMatMul (S/kernels/nvidia/basic_kernel_wrapper.cpp:1042-1052, cuBLASLt with scale pointers). */
size_t ksq_fp8_tensor_gemm_workspace_size(size_t max_m, size_t n, size_t k);
int ksq_fp8_tensor_gemm(const void* a_q, const void* a_scale, const void* b, const void* b_scale, void* out, size_t m,
                        size_t n, size_t k, int out_dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * W4A8: int4 weights (group 128 or 64, fp16 scales, no zero points) against statically quantized e4m3 activations,
 *   out[m,n] = T(alpha * sum_g scale[g,n] * sum_{k in g} a_q[m,k] * w[k,n]),  w in -8..7, fp32 accumulation.
 * The path of FinegrainedMixedDtypeGemmLayer (S/layers/nvidia/finegrained_mixed_dtype_gemm_layer.cpp:15-183) over
 * FinegrainedMixedDtypeGemmWrapper (K/gemm/finegrained_mixed_dtype_gemm/finegrained_mixed_dtype_gemm_wrapper.cpp).
 *
 * ksq_w4a8_repack_weight: src int8 [k, n/2], two's-complement nibbles, low nibble = even column - the tensor the
 *   reference gives to PreprocessWeightsForMixedGemm (S/models/weight_method/w4a8_awq_method.cpp:176-181) - into
 *   the 1 KiB fragment layout of the fp8 matrix instruction (n*k/2 bytes).  n % 16 == 0, k % 128 == 0.
 *   ksq_w4a8_unpack_weight is its inverse (bit-exact round trip).
 * ksq_w4a8_static_quant: q[m,k] = e4m3(x[m,k] / s), IEEE fp32 division, round to nearest even, saturating;
 *   s = scale[0] (KSQ_W4A8_PER_TENSOR), scale[channel] (KSQ_W4A8_PER_CHANNEL) or scale[row] (KSQ_W4A8_PER_TOKEN), fp32
 *   in device memory; and
 *   xsum[k/128, m] fp32 (group-major, tokens contiguous) = the sum of each group of 128 quantized values, which
 *   the GEMM needs.  KSQ_W4A8_SUMS_ONLY
 *   takes x that is e4m3 already and writes xsum only (q and scale unused).
 *   Replaces StaticQuantizeE4M3PerTensor / PerToken / PerChannel (wrapper.cpp:128-153 -> scaleMatrix,
 *   K/others/tensorrt-llm/dev/common/cudaFp8Utils.cu:38-52).
 * ksq_w4a8_gemm: a_q [m,k] e4m3 row-major, xsum [k/group,m], w_packed from ksq_w4a8_repack_weight, scales fp16
 *   [k/group, n] as the reference holds them (weight_scale / weight_scale_2), alpha = input_scale * weight_scale_2.
 *   Replaces FinegrainedMixedDtypeGemmWrapper::Forward (wrapper.cpp:68-100); no tactic argument: the kernel is
 *   chosen from the shape.
 * ------------------------------------------------------------------------------------------------------------------ */
enum { KSQ_W4A8_PER_TENSOR = 0, KSQ_W4A8_PER_CHANNEL = 1, KSQ_W4A8_SUMS_ONLY = 2, KSQ_W4A8_PER_TOKEN = 3,
       KSQ_W4A8_SUMS_PER_64 = 16 /* or-ed into the mode: xsum [k/64, m], one sum per 64 channels (GEMM group size 64) */ };
size_t ksq_w4a8_packed_weight_bytes(size_t n, size_t k);
int ksq_w4a8_repack_weight(const void* src, void* dst_packed, size_t n, size_t k, void* stream);
int ksq_w4a8_unpack_weight(const void* packed, void* dst, size_t n, size_t k, void* stream);
int ksq_w4a8_static_quant(const void* x, const void* scale, void* q, void* xsum, size_t m, size_t k, int mode,
                          int dtype, void* stream);
size_t ksq_w4a8_workspace_size(size_t max_m, size_t n, size_t k);
int ksq_w4a8_gemm(const void* a_q, const void* xsum, const void* w_packed, const void* scales, float alpha, void* out,
                  size_t m, size_t n, size_t k, size_t group, int out_dtype, void* workspace, size_t workspace_bytes,
                  void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * MoE: expert-offset / permutation build, grouped W4A16 GEMM, silu*mul, top-k sum.
 * ------------------------------------------------------------------------------------------------------------------ */

/* Counting sort of topk_ids[numel] (int32, ids outside [0,E) are dropped) by expert, every expert's segment padded
 * to a multiple of block_m with the value `numel`; order inside an expert is ascending flat index (deterministic,
 * unlike the atomic rank of sgl_moe_token_sort_kernel).  sorted_ids has ksq_moe_align_capacity() entries and is
 * completely written; expert_ids has capacity/block_m entries, num_post_pad one.  `scratch` is
 * ksq_moe_align_scratch_bytes() of device memory.
 * Replaces InvokeSglMoeAlignBlockSize / InvokeMoeAlignBlockSize / InvokeFillIntToBuffer
 * (K/moe_utils/moe_utils.cu:660-755). */
size_t ksq_moe_align_capacity(size_t numel, size_t E, size_t block_m);
size_t ksq_moe_align_scratch_bytes(size_t numel, size_t E);
int ksq_moe_align(const void* topk_ids, size_t numel, size_t E, size_t block_m, void* sorted_ids, void* expert_ids,
                  void* num_post_pad, void* scratch, void* stream);

/* Grouped GEMM over the aligned blocks: for every valid sorted slot id s (< numel)
 *   out[s, :] = x[s / top_k, :] . dequant(W[expert of s's block]) * (topk_w ? topk_w[s] : 1)
 * x [rows, k] T, out [numel, n] T, W/scales packed per expert as by ksq_w4a16_repack(E = experts),
 * zeros_packed NULL for symmetric (code-8).  top_k = 1 reads x rows by slot (second MoE GEMM).
 * block_m is the block size the permutation was aligned with: 16 or 32 run the streaming (decode) kernel, 128 or 256
 * the MFMA tile kernel (which multiplies only the 16-row tiles of a block that hold rows); ksq_moe_block_m() gives the
 * choice for a problem size.
 * A handful of slots (numel <= 64, block_m 16) need no aligned permutation: with sorted_ids NULL, expert_ids is the
 * router's topk_ids [numel] itself, num_post_pad is not read, and every slot is a block of its own (a slot whose id is
 * outside [0, E) leaves its output row unwritten, as the alignment would have dropped it).  One launch fewer in front
 * of a GEMM that takes tens of microseconds.
 * Replaces InvokeMoeWna16Gemm (K/moe/moe_wna16/moe_wna16.cu:263-288) and the Triton
 * InvokeFusedMoeGptqAwqKernel (S/kernels/nvidia/triton_wrapper.h:68-75). */
size_t ksq_moe_block_m(size_t numel, size_t E);
int ksq_moe_w4a16_gemm(void* out, const void* x, const void* w_packed, const void* scales_packed,
                       const void* zeros_packed, const void* topk_w, const void* sorted_ids, const void* expert_ids,
                       const void* num_post_pad, size_t numel, size_t top_k, size_t E, size_t n, size_t k,
                       size_t group, size_t block_m, int dtype, void* stream);

/* The first MoE GEMM with the activation in its epilogue: w_packed holds [gate | up] rows (n = 2 * inter), and for every
 * valid sorted slot id s   out[s, c] = T(silu(T(g)) * T(u)),  g = x[s / top_k, :] . W[e, c, :],  u = x[s / top_k, :] . W[e, inter + c, :],
 * out [numel, inter] T: bit for bit what ksq_moe_w4a16_gemm into a [numel, 2 * inter] buffer followed by ksq_silu_mul
 * gives, in one launch and without that buffer.  block_m 16, 32, 128 or 256, as for ksq_moe_w4a16_gemm (sorted_ids NULL
 * likewise).
 * Replaces the pair InvokeMoeWna16Gemm + InvokeSiluAndMul of InvokeFusedMoe
 * (S/kernels/nvidia/moe_kernel_wrapper.cpp:616-640). */
int ksq_moe_w4a16_gate_up_silu(void* out, const void* x, const void* w_packed, const void* scales_packed,
                               const void* zeros_packed, const void* sorted_ids, const void* expert_ids,
                               const void* num_post_pad, size_t numel, size_t top_k, size_t E, size_t n, size_t k,
                               size_t group, size_t block_m, int dtype, void* stream);

/* The second MoE GEMM and the sum over top-k in one launch, for up to 8 tokens:
 *   out[t, :] = T( sum_j topk_w[t, j] * (x[t * top_k + j, :] . dequant(W[topk_ids[t, j]])) ),  summed in fp32 and rounded once
 * x [tokens * top_k, k] T (the activation's output, a token's top_k rows one behind the other), out [tokens, n] T,
 * topk_w fp32 and topk_ids int32 [tokens, top_k] as the router wrote them (an id outside [0, E) contributes nothing).
 * A token's row block streams its top_k experts' weights as one long K; no aligned permutation, no [numel, n] buffer,
 * no separate sum (whose per-expert rounding to T this form does not have: it is closer to the fp32 reference).
 * Replaces InvokeMoeWna16Gemm followed by InvokeMoeSum for the decode steps of a few sequences
 * (K/moe/moe_wna16/moe_wna16.cu:36-217, which adds its partial results into the output with atomicAdd;
 * K/moe_utils/moe_utils.cu:789-835). */
int ksq_moe_w4a16_down_sum(void* out, const void* x, const void* w_packed, const void* scales_packed, const void* topk_w,
                           const void* topk_ids, size_t tokens, size_t top_k, size_t E, size_t n, size_t k, size_t group,
                           int dtype, void* stream);

/* Grouped blockwise-FP8 GEMM over the aligned blocks: for every valid sorted slot id s (< numel)
 *   out[s, :] = sum_kb (a_q[s / top_k, kb] . b[e, :, kb]) * a_s[kb, s / top_k] * b_s[e, :/128, kb] * (topk_w ? topk_w[s] : 1)
 * with e the expert of s's block.  a_q [a_rows, k] e4m3, a_s fp32 [a_rows, k/128] (the reference's layout) or, when
 * a_s_column_major, [k/128, a_rows] - the two layouts ksq_fp8_group_quant writes; b [E, n, k] e4m3 packed by
 * ksq_fp8_repack_weight(E = experts), b_s fp32 [E, ceil(n/128), k/128] as in the checkpoint, out [numel, n] in out_dtype.  top_k = 1 reads a_q rows by slot (second MoE GEMM).
 * block_m is the block size the permutation was aligned with: 16 or 32 run the streaming (decode) kernel, 128 or 256
 * the MFMA tile kernel; ksq_moe_fp8_block_m() gives the choice for a problem size.
 * Replaces the fp8_w8a8 block-quantized branch of InvokeFusedMoe's fused_moe_kernel launches
 * (S/kernels/nvidia/moe_kernel_wrapper.cpp:435-456, 498-522, 560-600). */
size_t ksq_moe_fp8_block_m(size_t numel, size_t E);
int ksq_moe_fp8_blockwise_gemm(void* out, const void* a_q, const void* a_s, int a_s_column_major, size_t a_rows, const void* b,
                               const void* b_s, const void* topk_w, const void* sorted_ids, const void* expert_ids,
                               const void* num_post_pad, size_t numel, size_t top_k, size_t E, size_t n, size_t k,
                               size_t block_m, int out_dtype, void* stream);
/* ksq_moe_w4a16_down_sum for block-quantized fp8 experts: the second GEMM and the sum over top-k in one launch, for up
 * to 8 tokens.  a_q [tokens * top_k, k] e4m3 with scales a_s [tokens * top_k, k/128] row-major (the second
 * quantization's output), b / b_s the experts' packed weights and block scales, topk_w / topk_ids [tokens, top_k];
 * out [tokens, n], the fp32 sum over a token's experts rounded once.  sorted_ids NULL in ksq_moe_fp8_blockwise_gemm is
 * the matching form of the first GEMM (block_m 16, at most 64 slots, expert_ids = topk_ids).
 * Replaces the fused_moe_kernel launch + InvokeMoeSum pair of InvokeFusedMoe for the decode steps of a few sequences
 * (S/kernels/nvidia/moe_kernel_wrapper.cpp:435-456, 640-652). */
int ksq_moe_fp8_down_sum(void* out, const void* a_q, const void* a_s, const void* b, const void* b_s, const void* topk_w,
                         const void* topk_ids, size_t tokens, size_t top_k, size_t E, size_t n, size_t k, int out_dtype,
                         void* stream);


/* Router: softmax over the E gating logits of every token in fp32, the top_k largest probabilities in descending
 * order (ties: lower expert id first), weights = probability * routed_scaling_factor, optionally renormalised to
 * sum to routed_scaling_factor over the top_k first (norm_topk_prob).  gating [tokens, E] in `dtype` (KSQ_F32
 * allowed), topk_w fp32 [tokens, top_k], topk_ids int32 [tokens, top_k].  E <= 1024, top_k <= 32.
 * Replaces InvokeBasicSoftmaxTopk (K/grouped_topk/grouped_topk.cu:678-755), the routing step in front of the path. */
int ksq_moe_topk_softmax(const void* gating, void* topk_w, void* topk_ids, size_t tokens, size_t E, size_t top_k,
                         int norm_topk_prob, float routed_scaling_factor, int dtype, void* stream);

/* Grouped router (DeepSeek-V2/V3 style).  Per token, in fp32:
 *   score  = softmax(gating) (KSQ_SCORE_SOFTMAX) or 1 / (1 + expf(-gating)) (KSQ_SCORE_SIGMOID)
 *   choose = score + e_bias[expert] when e_bias (fp32 [E]) is given, else score
 *   the E experts form num_expert_group equal groups; a group ranks by the sum of its two largest choose values
 *   (e_bias given) or by its largest (e_bias NULL); the topk_group best groups are kept (ties: lower group first)
 *   the top_k largest choose values among the kept groups select the experts (descending; ties: lower id first)
 *   weight = score of the selected expert (never the biased value), / sum over the top_k when renormalize,
 *   * routed_scaling_factor.
 * num_expert_group = topk_group = 1 with e_bias NULL is plain top-k routing with either scoring function.
 * E <= 1024 and a multiple of num_expert_group <= 64, top_k <= min(32, topk_group * E / num_expert_group).
 * Replaces InvokeGroupedTopk (S/kernels/nvidia/moe_kernel_wrapper.cpp:264-347: the fused sigmoid + bias form and
 * the general tensor-op form) and InvokeDeepSeekV3GroupedTopk (K/grouped_topk/grouped_topk.cu:507-665). */
#define KSQ_SCORE_SOFTMAX 0
#define KSQ_SCORE_SIGMOID 1
int ksq_moe_grouped_topk(const void* gating, const void* e_bias, void* topk_w, void* topk_ids, size_t tokens, size_t E,
                         size_t top_k, size_t num_expert_group, size_t topk_group, int scoring, int renormalize,
                         float routed_scaling_factor, int dtype, void* stream);

/* out[r, i] = T(silu(x[r, i]) * x[r, inter + i]), fp32 math a / (1 + expf(-a)) * b.
 * Replaces InvokeSiluAndMul (K/moe_utils/moe_utils.cu:893-905). */
int ksq_moe_silu_mul(const void* x, void* out, size_t rows, size_t inter, int dtype, void* stream);

/* out[t, :] = sum_j in[t, j, :], accumulated in T precision in ascending j.
 * Replaces InvokeMoeSum (K/moe_utils/moe_utils.cu:789-835). */
int ksq_moe_sum(const void* in, void* out, size_t tokens, size_t topk, size_t d, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------------------------------
 * Per-shape tile selection: a pure host function of (kind, m, n, k, dtype); no timing, no device access.
 * Replaces GetBestConfigIndex (K/asymmetric_gemm/asymmetric_gemm_wrapper.cu:101-146), machete_best_schedule
 * (K/machete/machete_wrapper.h:38-109), get_best_gemm_config (K/others/tensorrt-llm/dev/deep_gemm/jit_utils.cuh:143-222)
 * and the threshold sweep of BlockwiseMatMulLayer::Preprocess (S/layers/nvidia/blockwise_matmul_layer.cpp:71-181).
 * ------------------------------------------------------------------------------------------------------------------ */
enum { KSQ_KIND_W4A16 = 0, KSQ_KIND_FP8_BLOCKWISE = 1, KSQ_KIND_MOE_W4A16 = 2, KSQ_KIND_W4A8 = 3 };
enum { KSQ_KERNEL_SPLITK_WAVE = 0, KSQ_KERNEL_MFMA_TILE = 1 };

typedef struct ksq_tile_desc {
  int32_t kernel;   /* KSQ_KERNEL_* */
  int32_t block_m;  /* rows of x / tokens per workgroup */
  int32_t block_n;  /* output columns per workgroup */
  int32_t block_k;  /* k extent of one main-loop stage */
  int32_t waves;    /* wavefronts (64 lanes) per workgroup */
  int32_t split_k;  /* k slices reduced inside the kernel (across wavefronts and/or workgroups) */
  int32_t grid;     /* workgroups launched */
  int32_t x_chunk;  /* split-K wavefront kernel: k-tiles of activations staged through LDS at a time; 0 = through registers */
} ksq_tile_desc;

/* The descriptor describes group size 128.  Other group sizes of W4A16 keep the kernel and block shape but carry more
 * scales per k-tile; W4A8 with group 64 runs 128-token tiles whose K range is not cut (split_k and grid then differ
 * from what is reported here). */
int ksq_select_tile(int kind, size_t m, size_t n, size_t k, int dtype, ksq_tile_desc* out_desc);

/* Above 32 rows ksq_w4a16_gemm, ksq_fp8_blockwise_gemm and ksq_w4a8_gemm run the MFMA tile kernels, but for small
 * problems of up to 512 rows: while ceil(m / 32) * n * k <= 2^28 (W4A16 with group 128; 2^27 when k >= 4 n), or
 * <= 5 * 2^24 (block-fp8, n <= 4 k), or <= 5 * 2^25 (W4A8, n <= 4 k), the decode-form kernel over blocks of 32 rows is
 * faster (the tile kernels have a floor of about 20 us) and is what runs.  enabled = 0 switches that rule off for the whole process -
 * every m > 32 then runs the tile kernel -, 1 (the default) back on; returns the previous setting.  For tests that
 * must reach the tile kernels at sizes a CPU reference can multiply, and for timing one kernel against the other;
 * ksq_select_tile follows the setting, the workspace queries cover both settings.
 * No counterpart in the reference (its Marlin / CUTLASS / DeepGEMM paths have no such switch). */
int ksq_set_small_problem_rule(int enabled);

/* Measurement aid, no counterpart in the reference: one launch of 256 workgroups x 8 wavefronts, each issuing `iters`
 * rounds of independent matrix instructions on operands that stay in registers (no memory traffic, no LDS, no other
 * arithmetic).  kind 0 / 1 / 2: v_mfma_f32_16x16x32_f16 / _bf16 / v_mfma_scale_f32_16x16x128_f8f6f4 on e4m3 bytes, the
 * forms the GEMM kernels use; 3 / 4 / 5: the 32x32x16 and 32x32x64 forms of the same types.  constant_operands = 0:
 * every lane's operand bits differ; 1: all operands one value.  Timed by the caller (bench.py --mfma-stream), the rate
 * it sustains is what the matrix pipes deliver under the part's power limit - the ceiling a GEMM kernel on such data has
 * below the peak figure.  sink: 256 * 512 floats of device memory (never written for these operands).
 * ksq_diag_mfma_stream_flops: the floating-point operations of one such launch. */
int ksq_diag_mfma_stream(int kind, int constant_operands, int iters, void* sink, void* stream);
double ksq_diag_mfma_stream_flops(int kind, int iters);

#ifdef __cplusplus
}
#endif
#endif /* KSQ_H_ */
