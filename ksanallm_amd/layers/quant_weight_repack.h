// Loader-side half of the path: turns the tensors a GPTQ / AWQ checkpoint holds into the single packed weight tensor
// the layers consume, with its scale / zero-point tensors bound as side tensors.
// Stands where the reference converts layouts after slicing for tensor parallelism:
//   dense   QuantWeight::ConvertGroupTensor / PackAndBindGroupTensor  (src/ksana_llm/models/quant/quant_weight.cpp:321-520,
//           716-753) with CutlassUtils / MarlinUtils / MacheteUtils    (src/ksana_llm/models/quant/*_utils.cpp)
//   experts the [E, N, K/2] uint4x2 stacks of the moe-int4 loader      (src/ksana_llm/models/quant/quant_weight.cpp:182-319)
// All device work is enqueued on `stream`; the sources may be released once the stream has drained.
#pragma once

#include "base_layer.h"

namespace ksana_llm {

// qweight: GPTQ [K/8, N] int32 or AWQ [K, N/8] int32 (device).  scales: [K/group, N] in T.  qzeros: AWQ only,
// [K/group, N/8] int32 (nullptr for GPTQ, whose symmetric zero point 8 is implicit).
// g_idx: GPTQ act-order only, int32 [K] (device): quantization group of every input channel.  The rows are then
// packed in the order perm = stable argsort(g_idx) (MarlinSortGIdx, src/ksana_llm/models/quant/marlin_utils.cpp:106-122;
// computed on the host, which synchronizes `stream`) and `perm` and the sorted `g_idx` are bound to the result.
// Returns a TYPE_I4_GROUP tensor of logical shape {K, N/2} with `scales` (and `zeros`) bound.
// k_full = false (with g_idx): the tensors are a tensor-parallel rank's K range of an act-order checkpoint
// (row-parallel projection): qweight holds the rank's K rows, g_idx their checkpoint-wide group numbers and scales the
// scales of ALL groups, [G_total, N].  The rows are sorted by group, every run of equal group padded to a multiple of
// 32 rows; the result has shape {K', N/2}, K' >= K a multiple of 128, `scales` [K'/32, N] (one row per 32 packed rows:
// the layer runs it with group size 32), `perm` [K'] (-1 for padding rows) and the sorted `g_idx`.
Tensor PackGroupQuantWeight(const Tensor& qweight, const Tensor& scales, const Tensor* qzeros, QuantMode method,
                            size_t group_size, int rank, hipStream_t stream, const Tensor* g_idx = nullptr,
                            bool k_full = true);

// experts: [E, N, K/2] uint8, low nibble = even k.  scales: [E, N, K/group] in T.
// Returns a TYPE_UINT8 tensor of logical shape {E, N, K/2} (dtype and shape of the reference's moe-int4 stacks, which
// MoeLayerFactory::AutoCreateMoeLayer reads) with `scales` bound.
Tensor PackMoeExpertWeight(const Tensor& experts, const Tensor& scales, size_t group_size, int rank, hipStream_t stream);

// GPTQ expert stack as the Marlin MoE loader holds it before its own repack: qweight [E, K/8, N] int32, scales
// [E, K/group, N] in T (symmetric).  Returns a TYPE_INT32 tensor of logical shape {E, K/16, 2*N} (the shape the
// reference's Marlin repack gives, which AutoCreateMoeLayer derives the hidden size from) with `scales` bound, holding
// the same packed tiles PackMoeExpertWeight produces, for MarlinMoeLayer.  With g_idx (int32 [E, K], the checkpoint's
// act-order group index of every expert) each expert's rows are sorted by group and `perm` / the sorted `g_idx`
// ([E, K] each) are bound, as the reference binds them for fused_marlin_moe (S/layers/nvidia/marlin_moe_layer.cpp:71-81).
Tensor PackGptqExpertWeight(const Tensor& qweight, const Tensor& scales, size_t group_size, int rank, hipStream_t stream,
                            const Tensor* g_idx = nullptr);

// FP8 (e4m3) weights, [N, K] or an expert stack [E, N, K] in checkpoint layout: returns the same shape and dtype in the
// packed 2 KiB fragment layout every FP8 layer here consumes (BlockwiseMatMulLayer, Fp8MatMulLayer, MoeLayer with
// block-fp8 experts); the side tensors of `weight` (weight_scales, input_scales, ...) are carried over unchanged.
// Stands where the reference binds the scales of FP8 weights after loading (quant_weight.cpp:817-861).
Tensor PackFp8Weight(const Tensor& weight, int rank, hipStream_t stream);

// W4A8 weight as the reference holds it before PreprocessWeightsForMixedGemm
// (src/ksana_llm/models/weight_method/w4a8_awq_method.cpp:158-181): [K, N/2] bytes, two's-complement nibbles, low
// nibble = even column -> the packed fragment layout FinegrainedMixedDtypeGemmLayer consumes.  The tensor keeps its
// shape; input_scales, weight_scales, pre_quant_scales and alpha are carried over.
Tensor PackW4A8Weight(const Tensor& weight, int rank, hipStream_t stream);

}  // namespace ksana_llm
