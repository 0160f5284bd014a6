// W4A8 matmul layer: int4 group-128 weights (fp16 scales) against activations quantized to e4m3 with the checkpoint's
// static scale.  Mirrors src/ksana_llm/layers/finegrained_mixed_dtype_gemm_layer.h:15-77 and
// nvidia/finegrained_mixed_dtype_gemm_layer.cpp:15-183: the same parameter struct, the same workspace order
// ([kernel scratch][m*k quantized activations]) with the per-group activation sums the kernel needs appended, the same
// side tensors of the weight (input_scales, weight_scales, pre_quant_scales, alpha).  The reference's Preprocess times
// every CUTLASS tactic for every token count up to max_batch_size; here the kernel follows from the shape, so
// Preprocess only checks that one exists.
#pragma once

#include "base_layer.h"

namespace ksana_llm {

#ifndef KSQ_IN_KSANA_TREE
struct FinegrainedMixedDtypeGemmLayerParameters : public BaseLayerParameters {
  size_t m{0};
  size_t n{0};
  size_t k{0};
  size_t group_size{0};
  bool has_zero{false};
  DataType activation_type{TYPE_INVALID};
  DataType output_type{TYPE_INVALID};
};
#endif

class FinegrainedMixedDtypeGemmLayer : public BaseLayer {
 public:
  // parameters: one FinegrainedMixedDtypeGemmLayerParameters
  Status Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
              std::shared_ptr<Context> context, int rank) override;
  size_t GetWorkspaceSize() override;
  Status Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) override;
  // inputs: [0] activations [m, k] T; [1] weight packed by PackW4A8Weight (quant_weight_repack.h), shape [k, n/2], with
  // weight_scales (fp16 [k/128, n]), alpha, and input_scales (1 fp32) or pre_quant_scales (fp32 [k], the per-channel
  // divisor input_scale / pre_quant_scale).  output [0]: [m, n] in T.
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;

 private:
  FinegrainedMixedDtypeGemmLayerParameters params_;
  size_t kernel_workspace_size_ = 0;
  size_t quantized_size_ = 0;
  size_t sums_size_ = 0;
};

}  // namespace ksana_llm
