// GPTQ int4 experts behind the reference's Marlin MoE layer interface ("hunyuan-large int4":
// src/ksana_llm/layers/marlin_moe_layer.h:13-52, nvidia/marlin_moe_layer.cpp:10-104, and the sequence of
// fused_marlin_moe, 3rdparty/LLM_kernels/csrc/kernels/nvidia/marlin_moe/fused_marlin_moe.cu:74-207):
//   softmax top-k over the gating output (renormalized when the norm mode says so) -> align -> grouped GEMM gate_up ->
//   silu*mul -> grouped GEMM down (x routing weight) -> sum over top-k.
// That is the sequence MoeLayer runs for int4 experts, on the same kernels; what differs is the interface: 20 init
// parameters (no layer index), fp16 activations only, and no grouped / sigmoid routing.  The weights are the expert
// stacks packed by PackMoeExpertWeight (where the reference holds Marlin tiles), with their scales bound.
// Act-order experts (perm bound to a weight by PackGptqExpertWeight) run with one extra pass per GEMM that gathers every
// slot's activation row through its expert's permutation; zero points are rejected with a message.
#pragma once

#include "moe_layer.h"

namespace ksana_llm {

class MarlinMoeLayer : public MoeLayer {
 public:
  // parameters (the reference's 20 positional values):
  //   MoeScaleNormMode, size_t max_token_num, size_t expert_num, size_t expert_hidden_size, size_t expert_inter_size,
  //   size_t expert_topk, size_t tp_size, bool use_vllm_moe, uint32_t num_expert_group, uint32_t expert_groups_topk,
  //   std::string scoring_func, std::string topk_method, bool norm_topk_prob, float routed_scaling_factor,
  //   bool use_e_score_correction_bias, bool enable_full_shared_expert, DataType fp8_weight_dtype,
  //   DataType int_weight_dtype, int group_size, bool apply_weight
  Status Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
              std::shared_ptr<Context> context, int rank) override;
  // inputs as for MoeLayer: [0] hidden_states fp16, [1] gating_output [tokens, experts] fp16 (or fp32),
  // [2] up_gate weight, [3] down weight.  Anything but fp16 hidden states throws, as in the reference.
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;
};

}  // namespace ksana_llm
