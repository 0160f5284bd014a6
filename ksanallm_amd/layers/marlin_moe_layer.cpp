#include "marlin_moe_layer.h"

namespace ksana_llm {

Status MarlinMoeLayer::Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
                            std::shared_ptr<Context> context, int rank) {
  if (parameters.size() < 20) return Status(RET_INVALID_ARGUMENT, "MarlinMoeLayer: expects 20 init parameters");
  // the same values in MoeLayer's order.  The reference's Init reads 20 values without a layer index
  // (marlin_moe_layer.cpp:17-36), while its factory's vector carries the layer index as third value
  // (moe_layer_factory.cpp:150-151): both orders are accepted, told apart by the type of the third value.
  std::vector<std::any> p;
  if (parameters.size() >= 21 && parameters[2].type() == typeid(int)) {
    p.assign(parameters.begin(), parameters.begin() + 21);
  } else {
    p.assign(parameters.begin(), parameters.begin() + 2);
    p.push_back(static_cast<int>(0));
    p.insert(p.end(), parameters.begin() + 2, parameters.begin() + 20);
  }
  // fused_marlin_moe routes with a plain softmax top-k whatever the routing fields say, and never scales the weights
  p[9] = static_cast<uint32_t>(1);    // num_expert_group
  p[10] = static_cast<uint32_t>(1);   // expert_groups_topk
  p[11] = std::string("softmax");     // scoring_func
  p[12] = std::string("greedy");      // topk_method
  // norm_topk_prob: in this layer the norm mode alone decides (fused_marlin_moe takes it, marlin_moe_layer.cpp:91-95)
  p[13] = std::any_cast<const MoeScaleNormMode>(parameters[0]) == MoeScaleNormMode::RE_NORM;
  p[14] = 1.0f;                       // routed_scaling_factor
  p[15] = false;                      // use_e_score_correction_bias
  p[8] = true;                        // the aligned-block flow is the only one here
  if (std::any_cast<DataType>(p[17]) != TYPE_INVALID)
    return Status(RET_INVALID_ARGUMENT, "MarlinMoeLayer: fp8 expert weights do not belong to this layer");
  p[18] = TYPE_UINT4x2;               // int_weight_dtype: 4-bit codes, two per byte
  if (runtime_config.inter_data_type != TYPE_FP16)
    return Status(RET_INVALID_ARGUMENT, "MarlinMoeLayer: only fp16 activations (marlin_moe_layer.cpp:96-99)");
  reserve_act_order_ = true;  // g_idx / perm may come bound to the weights (marlin_moe_layer.cpp:71-81)
  return MoeLayer::Init(p, runtime_config, context, rank);
}

Status MarlinMoeLayer::Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) {
  if (input_tensors.size() < 4) KLLM_THROW("MarlinMoeLayer: expects hidden_states, gating_output, up_gate weight, down weight");
  if (input_tensors[0].dtype != TYPE_FP16) {
    KLLM_THROW("marlin moe only support input type " + std::to_string(TYPE_FP16) + ", not support input type " +
               std::to_string(input_tensors[0].dtype));
  }
  for (int i : {2, 3}) {
    if (input_tensors[i].GetPtr<void>() == nullptr) KLLM_THROW("w1 or w2 is nullptr.");
    if (!input_tensors[i].scales || input_tensors[i].scales->GetPtr<void>() == nullptr)
      KLLM_THROW("w1_scales or w2_scales is nullptr.");
    if (input_tensors[i].g_idx && !input_tensors[i].perm)
      KLLM_THROW("MarlinMoeLayer: g_idx without perm: pack act-order experts with PackGptqExpertWeight");
    if (input_tensors[i].zeros) KLLM_THROW("MarlinMoeLayer: expert zero points are not built");
  }
  // hidden_states, gating_output, w1, w2 only: the router of this layer takes no bias and no expert map
  std::vector<Tensor> inputs(input_tensors.begin(), input_tensors.begin() + 4);
  return MoeLayer::Forward(inputs, output_tensors);
}

}  // namespace ksana_llm
