// Fused MoE layer for int4 group-quantized experts (the "moe-int4" path: weights [E, N, K/2] uint4x2 with per-group
// scales, activations in T) and for block-quantized fp8 experts (weights [E, N, K] e4m3 with fp32 scales per 128 x 128
// block bound as weight_scales, packed by PackFp8Weight; activations quantized per token and 128 channels in front of
// each GEMM).  Mirrors src/ksana_llm/layers/moe_layer.h:42 and nvidia/moe_layer.cpp:38-380 together with
// InvokeFusedMoe (src/ksana_llm/kernels/nvidia/moe_kernel_wrapper.cpp:466-657):
//   router (softmax top-k, or grouped / sigmoid / bias-corrected top-k with the bias as input tensor 5) -> align/permute -> grouped GEMM gate_up -> silu*mul -> grouped GEMM down (x routing
//   weight) -> sum over top-k, processed in chunks of 32768 tokens, all scratch carved out of one workspace buffer.
// Expert parallelism, DeepEP, EPLB and the per-tensor fp8 / w4afp8 weight types of the reference class are not part of this path
// and make Init fail with a message.
#pragma once

#include "base_layer.h"

namespace ksana_llm {

class MoeLayer : public BaseLayer {
 public:
  // parameters (same 21 positional values as the reference):
  //   MoeScaleNormMode, size_t max_token_num, int layer_idx, size_t expert_num, size_t expert_hidden_size,
  //   size_t expert_inter_size, size_t expert_topk, size_t tp_size, bool use_vllm_moe, uint32_t num_expert_group,
  //   uint32_t expert_groups_topk, std::string scoring_func, std::string topk_method, bool norm_topk_prob,
  //   float routed_scaling_factor, bool use_e_score_correction_bias, bool enable_full_shared_expert,
  //   DataType fp8_weight_dtype, DataType int_weight_dtype, int group_size, bool apply_weight
  Status Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
              std::shared_ptr<Context> context, int rank) override;
  size_t GetWorkspaceSize() override;
  Status SetWorkspaceBuffer(const std::shared_ptr<Tensor>& workspace_buffer) override;
  Status Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) override;
  // inputs: [0] hidden_states [tokens, hidden] T, [1] gating_output [tokens, experts] T (or fp32),
  //         [2] up_gate_proj weight (packed, N = 2*inter, K = hidden) with scales bound,
  //         [3] down_proj weight (packed, N = hidden, K = inter) with scales bound.
  // output [0]: [tokens, hidden] T.
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;

  // rows per expert block for a chunk (InvokeFusedMoe picks 16 / 32 / 64 by token count; here the library decides by
  // rows per expert, which changes no result)
  size_t BlockM(size_t tokens) const {
    if (IsFp8()) return ksq_moe_fp8_block_m(tokens * expert_topk_, expert_num_per_node_);
    return ksq_moe_block_m(tokens * expert_topk_, expert_num_per_node_);
  }
  bool IsFp8() const { return compute_dtype_ == TYPE_BLOCK_FP8_E4M3; }

 protected:
  // act-order experts (weights with `perm` bound): the activation rows of every slot are gathered through its expert's
  // permutation in front of each GEMM, into workspace that is reserved only when a derived layer asks for it before
  // Init (MarlinMoeLayer does)
  bool reserve_act_order_ = false;

 private:
  static constexpr size_t kChunk = 32 * 1024;
  // up to this many tokens the int4 block runs its two-launch form: every slot a block of its own in the first GEMM,
  // the sum over top-k inside the second (ksq_moe_w4a16_down_sum).  DeepSeek-V3 expert shapes, whole block with /
  // without it: 1 token 39.5 / 49.5 us, 2 68 / 74, 4 128 / 135, 8 230 / 211
  static constexpr size_t kFewTokens = 4;

  MoeScaleNormMode moe_scale_norm_mode_ = MoeScaleNormMode::NO_NORM;
  size_t max_token_num_ = 0;
  int layer_idx_ = 0;
  size_t expert_num_per_node_ = 0;
  size_t expert_hidden_size_ = 0;
  size_t expert_inter_size_ = 0;
  size_t expert_topk_ = 0;
  bool use_vllm_moe_ = true;
  uint32_t num_expert_group_ = 1;
  uint32_t expert_groups_topk_ = 1;
  std::string scoring_func_ = "softmax";
  std::string topk_method_ = "greedy";
  bool norm_topk_prob_ = false;
  float routed_scaling_factor_ = 1.0f;
  bool use_e_score_correction_bias_ = false;
  bool apply_weight_ = false;
  DataType weight_dtype_ = TYPE_INVALID;
  DataType compute_dtype_ = TYPE_INVALID;
  int group_size_ = 128;

  // workspace carve-up (byte sizes, 256-aligned like the reference's AlignAddress)
  size_t topk_weights_size_ = 0, topk_ids_size_ = 0, fused_id_buffer_size_ = 0, align_scratch_size_ = 0;
  size_t cache1_size_ = 0, cache2_size_ = 0, cache3_size_ = 0, cache13_size_ = 0;
  size_t a1_q_size_ = 0, a1_size_ = 0, a2_q_size_ = 0;  // block-fp8: quantized activations
  size_t act_order1_size_ = 0, act_order2_size_ = 0;
  size_t max_ws_bytes_ = 0;
};

}  // namespace ksana_llm
