#include "layer_factory.h"

#include "blockwise_matmul_layer.h"
#include "finegrained_mixed_dtype_gemm_layer.h"
#include "fp8_matmul_layer.h"
#include "moe_layer.h"
#include "marlin_moe_layer.h"
#include "w4a16_matmul_layer.h"

namespace ksana_llm {

MatMulLayerFactory::MatMulLayerFactory(const ModelConfig& model_config, const RuntimeConfig& runtime_config,
                                       const int rank, std::shared_ptr<Context> context)
    : context_(context), rank_(rank), model_config_(model_config), runtime_config_(runtime_config) {
  for (DataType t : {TYPE_FP16, TYPE_BF16}) {
    // the reference registers both quant modes under the same classes; AWQ-vs-GPTQ travels in the init parameters
    for (QuantMode q : {QUANT_GPTQ, QUANT_AWQ}) {
      builder_map_[{TYPE_I4_GROUP, t, t, q, CUTLASS_LINEAR_BACKEND}] = &MatMulLayerFactory::BuildLayer<CutlassMatMulLayer>;
      builder_map_[{TYPE_I4_GROUP, t, t, q, MARLIN_LINEAR_BACKEND}] = &MatMulLayerFactory::BuildLayer<MarlinMatMulLayer>;
      builder_map_[{TYPE_I4_GROUP, t, t, q, MACHETE_LINEAR_BACKEND}] = &MatMulLayerFactory::BuildLayer<MacheteMatMulLayer>;
    }
    builder_map_[{TYPE_I4_GROUP, t, t, QUANT_W4A8_AWQ, CUTLASS_LINEAR_BACKEND}] =
        &MatMulLayerFactory::BuildLayer<FinegrainedMixedDtypeGemmLayer>;
    builder_map_[{TYPE_FP8_E4M3, t, t, QUANT_BLOCK_FP8_E4M3, DEFAULT_LINEAR_BACKEND}] =
        &MatMulLayerFactory::BuildLayer<BlockwiseMatMulLayer>;
    builder_map_[{TYPE_FP8_E4M3, t, t, QUANT_FP8_E4M3, DEFAULT_LINEAR_BACKEND}] = &MatMulLayerFactory::BuildLayer<Fp8MatMulLayer>;
  }
  // fp32 activations: the two fp8 layers, as in the reference's map (matmul_layer_factory.cpp:70-71, 77-78)
  builder_map_[{TYPE_FP8_E4M3, TYPE_FP32, TYPE_FP32, QUANT_BLOCK_FP8_E4M3, DEFAULT_LINEAR_BACKEND}] =
      &MatMulLayerFactory::BuildLayer<BlockwiseMatMulLayer>;
  builder_map_[{TYPE_FP8_E4M3, TYPE_FP32, TYPE_FP32, QUANT_FP8_E4M3, DEFAULT_LINEAR_BACKEND}] =
      &MatMulLayerFactory::BuildLayer<Fp8MatMulLayer>;
}

std::shared_ptr<BaseLayer> MatMulLayerFactory::CreateLayer(DataType weight_type, DataType input_type,
                                                           DataType output_type,
                                                           const std::vector<std::any>& init_params,
                                                           QuantMode quant_mode, LinearComputeBackend backend) {
  auto it = builder_map_.find({weight_type, input_type, output_type, quant_mode, backend});
  if (it == builder_map_.end()) {
    KLLM_THROW("Not support weight_type " + std::to_string(weight_type) + ", input_type " + std::to_string(input_type) +
               ", output_type " + std::to_string(output_type) + ", quant_mode " + std::to_string(quant_mode) +
               ", backend " + std::to_string(backend) + ".");
  }
  std::shared_ptr<BaseLayer> layer = (this->*(it->second))();
  Status status = layer->Init(init_params, runtime_config_, context_, rank_);
  if (!status.OK()) KLLM_THROW(status.GetMessage());
  return layer;
}

std::vector<std::any> MatMulLayerFactory::GroupMatMulParams(size_t n, size_t k, bool k_full) const {
  std::vector<std::any> p;
  p.push_back(runtime_config_.max_step_token_num);                                        // m
  p.push_back(n);                                                                         // n
  p.push_back(k);                                                                         // k
  p.push_back(model_config_.quant_config.group_size);                                     // groupsize
  p.push_back(static_cast<bool>(model_config_.quant_config.method == QUANT_AWQ));         // awq
  p.push_back(static_cast<bool>(model_config_.quant_config.desc_act));                    // gptq desc
  p.push_back(k_full);                                                                    // k full
  p.push_back(true);                                                                      // cuda gemv
  p.push_back(TYPE_I4_GROUP);                                                             // weight data type
  return p;
}

bool MatMulLayerFactory::ProjectionShape(const std::string& weight_name, size_t* k, size_t* n, bool* k_full) const {
  const auto& par = runtime_config_.parallel_basic_config;
  const bool full_shared = runtime_config_.enable_full_shared_expert;
  const size_t tp = full_shared ? 1 : par.tensor_parallel_size;
  const size_t attn_tp = par.attn_tensor_parallel_size;
  const size_t hidden = model_config_.hidden_units;
  size_t inter = model_config_.inter_size / tp;
  const size_t shared_inter = model_config_.moe_config.shared_expert_inter_size / tp;
  if (model_config_.type == "qwen") inter /= 2;  // that model's config.json states twice its inter size
  const MlaConfig& mla = model_config_.mla_config;
  const size_t heads = model_config_.head_num / attn_tp;
  const size_t qkv = model_config_.size_per_head * (model_config_.head_num + 2 * model_config_.num_key_value_heads);
  const size_t o_in = heads * (mla.v_head_dim > 0 ? mla.v_head_dim : model_config_.size_per_head);
  struct Row {
    const char* name;
    size_t k, n;
    bool k_full;
  };
  // column-parallel projections keep all of K on every rank; row-parallel ones (down / o) hold a slice of it
  const Row rows[] = {
      {"mlp.gate_proj", hidden, inter, true},
      {"mlp.up_proj", hidden, inter, true},
      {"mlp.down_proj", inter, hidden, false},
      {"mlp.shared_expert.gate_proj", hidden, shared_inter, true},
      {"mlp.shared_expert.up_proj", hidden, shared_inter, true},
      {"mlp.shared_expert.down_proj", shared_inter, hidden, false},
      {"query_key_value", hidden, qkv / attn_tp, true},
      {"q_proj", hidden, hidden / attn_tp, true},
      {"o_proj", o_in, hidden, false},
      // multi-head latent attention
      {"q_a_proj", hidden, mla.q_lora_rank, false},
      {"kv_a_lora_proj", hidden, mla.kv_lora_rank, false},
      {"kv_a_rope_proj", hidden, mla.qk_rope_head_dim, false},
      {"q_b_nope_proj", mla.q_lora_rank, heads * mla.qk_nope_head_dim, true},
      {"q_b_rope_proj", mla.q_lora_rank, heads * mla.qk_rope_head_dim, true},
      {"q_b_nope_rope_proj", mla.q_lora_rank, heads * (mla.qk_nope_head_dim + mla.qk_rope_head_dim), true},
      {"kv_b_nope_proj", mla.kv_lora_rank, heads * mla.qk_nope_head_dim, true},
      {"v_head_proj", mla.kv_lora_rank, heads * mla.v_head_dim, true},
  };
  for (const Row& r : rows) {
    if (weight_name.find(r.name) != std::string::npos) {
      *k = r.k;
      *n = r.n;
      *k_full = r.k_full;
      return true;
    }
  }
  return false;
}

std::shared_ptr<BaseLayer> MatMulLayerFactory::AutoCreateLayer(std::shared_ptr<BaseWeight> base_weight,
                                                               std::string weight_name, DataType weight_type,
                                                               DataType input_type, DataType output_type,
                                                               LinearComputeBackend backend,
                                                               const std::vector<std::any>& init_params) {
  (void)weight_type;
  // W4A8: the loader recorded the mode and the logical n, k with the weight
  const WeightStatus& status = context_->GetWeightStatus(weight_name);
  if (status.quant_mode == QUANT_W4A8_AWQ) {
    FinegrainedMixedDtypeGemmLayerParameters param;
    param.m = runtime_config_.max_step_token_num;
    param.n = status.layout.at("n");
    param.k = status.layout.at("k");
    param.group_size = 128;
    param.has_zero = false;
    param.activation_type = TYPE_FP8_E4M3;
    param.output_type = output_type;
    return CreateLayer(TYPE_I4_GROUP, input_type, output_type, {param}, QUANT_W4A8_AWQ, CUTLASS_LINEAR_BACKEND);
  }
  // GPTQ / AWQ group quantization: the shape comes from the projection's name
  const QuantMode method = model_config_.quant_config.method;
  if (model_config_.is_quant && (method == QUANT_GPTQ || method == QUANT_AWQ)) {
    size_t k = 0, n = 0;
    bool k_full = true;
    if (ProjectionShape(weight_name, &k, &n, &k_full)) {
      // (the reference creates every such layer under the GPTQ key; AWQ travels in the parameters.  kv_a_rope_proj is
      // too narrow for its other kernels and always takes the Marlin one.)
      const bool narrow = weight_name.find("kv_a_rope_proj") != std::string::npos;
      return CreateLayer(TYPE_I4_GROUP, input_type, output_type, GroupMatMulParams(n, k, k_full), QUANT_GPTQ,
                         narrow ? MARLIN_LINEAR_BACKEND : backend);
    }
  }
  // fp8 weights, [n, k]: blockwise scales or one scale per tensor
  const Tensor weight = base_weight->GetModelWeights(weight_name);
  if (weight.dtype == TYPE_FP8_E4M3) {
    if (weight.shape.size() != 2) KLLM_THROW("AutoCreateLayer: fp8 weight " + weight_name + " is not [n, k]");
    std::vector<std::any> p;
    p.push_back(runtime_config_.max_step_token_num);
    if (method == QUANT_BLOCK_FP8_E4M3) {
      p.push_back(size_t(weight.shape[0]));                                // n
      p.push_back(size_t(weight.shape[1]));                                // k
      p.push_back(model_config_.quant_config.weight_block_size.at(1));     // block size along k
      p.push_back(weight);
      p.insert(p.end(), init_params.begin(), init_params.end());           // skip_quant, layer type
      return CreateLayer(TYPE_FP8_E4M3, input_type, output_type, p, QUANT_BLOCK_FP8_E4M3, DEFAULT_LINEAR_BACKEND);
    }
    p.push_back(size_t(weight.shape[1]));                                  // k
    return CreateLayer(TYPE_FP8_E4M3, input_type, output_type, p, QUANT_FP8_E4M3, DEFAULT_LINEAR_BACKEND);
  }
  KLLM_THROW("AutoCreateLayer: " + weight_name + " is not a quantized weight; unquantized matmul layers stay with the host framework");
}

MoeLayerFactory::MoeLayerFactory(const ModelConfig& model_config, const RuntimeConfig& runtime_config, const int rank,
                                 std::shared_ptr<Context> context)
    : context_(context), rank_(rank), model_config_(model_config), runtime_config_(runtime_config) {
  // "deepseek moe-int4" rows of the reference
  builder_map_[{TYPE_UINT8, TYPE_FP16, TYPE_FP16, MOE_QUANT_GPTQ, TRITON_MOE_BACKEND}] = &MoeLayerFactory::BuildLayer<MoeLayer>;
  builder_map_[{TYPE_UINT8, TYPE_BF16, TYPE_BF16, MOE_QUANT_GPTQ, TRITON_MOE_BACKEND}] = &MoeLayerFactory::BuildLayer<MoeLayer>;
  // "hunyuan-large int4" row
  builder_map_[{TYPE_I4_GROUP, TYPE_FP16, TYPE_FP16, MOE_QUANT_GPTQ, MARLIN_MOE_BACKEND}] = &MoeLayerFactory::BuildLayer<MarlinMoeLayer>;
  // "deepseek fp8 blockwise" rows
  builder_map_[{TYPE_FP8_E4M3, TYPE_FP16, TYPE_FP16, MOE_QUANT_BLOCK_FP8_E4M3, TRITON_MOE_BACKEND}] = &MoeLayerFactory::BuildLayer<MoeLayer>;
  builder_map_[{TYPE_FP8_E4M3, TYPE_BF16, TYPE_BF16, MOE_QUANT_BLOCK_FP8_E4M3, TRITON_MOE_BACKEND}] = &MoeLayerFactory::BuildLayer<MoeLayer>;
}

std::shared_ptr<BaseLayer> MoeLayerFactory::CreateLayer(DataType weight_type, DataType input_type, DataType output_type,
                                                        const std::vector<std::any>& init_params, QuantMode quant_mode,
                                                        MoeComputeBackend backend) {
  auto it = builder_map_.find({weight_type, input_type, output_type, quant_mode, backend});
  if (it == builder_map_.end()) {
    KLLM_THROW("Not support weight_type " + std::to_string(weight_type) + ", input_type " + std::to_string(input_type) +
               ", output_type " + std::to_string(output_type) + ", quant_mode " + std::to_string(quant_mode) +
               ", moe backend " + std::to_string(backend) + ".");
  }
  std::shared_ptr<BaseLayer> layer = (this->*(it->second))();
  Status status = layer->Init(init_params, runtime_config_, context_, rank_);
  if (!status.OK()) KLLM_THROW(status.GetMessage());
  return layer;
}

}  // namespace ksana_llm

namespace ksana_llm {

std::shared_ptr<BaseLayer> MoeLayerFactory::AutoCreateMoeLayer(std::shared_ptr<BaseWeight> base_weight,
                                                               std::vector<std::string> weight_names,
                                                               DataType weight_type, DataType input_type,
                                                               DataType output_type, int layer_idx,
                                                               const std::vector<std::any>& init_params) {
  if (weight_names.size() < 2) KLLM_THROW("AutoCreateMoeLayer: expects the up_gate and the down expert weight names");
  const MoeConfig& moe = model_config_.moe_config;
  const QuantConfig& quant = model_config_.quant_config;
  const auto& par = runtime_config_.parallel_basic_config;
  const Tensor up_gate = base_weight->GetModelWeights(weight_names[0]);
  const Tensor down = base_weight->GetModelWeights(weight_names[1]);
  if (up_gate.shape.size() != 3 || down.shape.size() != 3) KLLM_THROW("AutoCreateMoeLayer: expert weights must be 3-D stacks");
  if (up_gate.shape[0] != down.shape[0]) {
    KLLM_THROW("up_gate experts " + std::to_string(up_gate.shape[0]) + " != down_experts " + std::to_string(down.shape[0]));
  }
  // int4 experts: a GPTQ 4-bit model, or an fp8 model whose first sub-configuration names these layers as GPTQ
  bool int4 = false;
  if (quant.method == QUANT_GPTQ && quant.bits == 4) {
    int4 = true;
  } else if (quant.method != QUANT_GPTQ && !model_config_.sub_quant_configs.empty() &&
             model_config_.sub_quant_configs[0].method == QUANT_GPTQ) {
    const QuantConfig& sub = model_config_.sub_quant_configs[0];
    for (const std::string& pattern : sub.pattern_layers) int4 = int4 || weight_names[0].find(pattern) != std::string::npos;
    for (const std::string& ignored : sub.ignored_layers) {
      if (weight_names[0].find(ignored) != std::string::npos) int4 = false;
    }
  }
  // both stacks must agree on the hidden size; packed layouts hide it behind their own factors
  size_t hidden_of_up_gate = up_gate.shape[2], hidden_of_down = down.shape[1];
  if (int4 && moe.use_vllm_moe) {
    hidden_of_up_gate = hidden_of_up_gate / 4 * (32 / quant.bits);  // [E, 2*inter, hidden / 2] bytes
  } else if (int4) {                                                // Marlin tiles: [E, k / 16, 2 * n] words
    hidden_of_up_gate = up_gate.shape[1] / (sizeof(int) / quant.bits) * 16;
    hidden_of_down = down.shape[2] / quant.bits * 2;
  }
  if (hidden_of_up_gate != hidden_of_down) {
    KLLM_THROW("up_gate_experts hidden_size != down_experts hidden_size " + std::to_string(hidden_of_up_gate) + " " +
               std::to_string(hidden_of_down));
  }
  weight_type = up_gate.dtype;
  if (down.dtype != weight_type) {
    KLLM_THROW("down_experts dtype " + std::to_string(down.dtype) + " != up_gate_experts dtype " + std::to_string(weight_type));
  }

  const size_t inter_per_rank = (moe.moe_inter_size + par.moe_tensor_para_size - 1) / par.moe_tensor_para_size;
  const size_t experts_per_node = moe.num_experts / (par.expert_parallel_size * par.expert_world_size);
  const bool block_fp8 = !int4 && quant.is_fp8_blockwise;
  DataType int_dtype = TYPE_INVALID;
  if (int4) int_dtype = weight_type == TYPE_UINT8 ? TYPE_UINT4x2 : (weight_type == TYPE_INT8 ? TYPE_INT4x2 : TYPE_I4_GROUP);

  std::vector<std::any> p = init_params;               // moe_scale_norm_mode
  p.push_back(runtime_config_.max_step_token_num);     // max_token_num
  p.push_back(layer_idx);
  p.push_back(experts_per_node);
  p.push_back(size_t(model_config_.hidden_units));
  p.push_back(inter_per_rank);
  p.push_back(moe.experts_topk);
  p.push_back(par.tensor_parallel_size);
  p.push_back(moe.use_vllm_moe);
  p.push_back(moe.num_expert_group);
  p.push_back(moe.expert_groups_topk);
  p.push_back(moe.scoring_func);
  p.push_back(moe.topk_method);
  p.push_back(moe.norm_topk_prob);
  p.push_back(moe.routed_scaling_factor);
  p.push_back(moe.use_e_score_correction_bias);
  p.push_back(runtime_config_.enable_full_shared_expert);
  p.push_back(block_fp8 ? TYPE_BLOCK_FP8_E4M3 : TYPE_INVALID);   // fp8_weight_dtype
  p.push_back(int_dtype);                                        // int_weight_dtype
  p.push_back(int4 ? static_cast<int>(quant.group_size) : 0);    // group_size
  p.push_back(moe.apply_weight);

  if (weight_type == TYPE_FP8_E4M3) {
    return quant.is_fp8_blockwise
               ? CreateLayer(weight_type, input_type, output_type, p, MOE_QUANT_BLOCK_FP8_E4M3, TRITON_MOE_BACKEND)
               : CreateLayer(weight_type, input_type, output_type, p, MOE_QUANT_FP8_E4M3, DEFAULT_MOE_BACKEND);
  }
  if (int4) {
    const bool triton_w4afp8 = runtime_config_.w4afp8_moe_backend == W4AFP8_MOE_BACKEND::GroupTriton ||
                               runtime_config_.w4afp8_moe_backend == W4AFP8_MOE_BACKEND::TensorTriton;
    if (weight_type == TYPE_UINT8 || triton_w4afp8)
      return CreateLayer(weight_type, input_type, output_type, p, MOE_QUANT_GPTQ, TRITON_MOE_BACKEND);
    if (weight_type == TYPE_INT8) return CreateLayer(weight_type, input_type, output_type, p, MOE_QUANT_GPTQ, CUTLASS_MOE_BACKEND);
    if (!moe.use_vllm_moe) return CreateLayer(TYPE_I4_GROUP, input_type, output_type, p, MOE_QUANT_GPTQ, MARLIN_MOE_BACKEND);
  }
  return CreateLayer(weight_type, input_type, output_type, p, MOE_QUANT_NONE, DEFAULT_MOE_BACKEND);
}

}  // namespace ksana_llm
