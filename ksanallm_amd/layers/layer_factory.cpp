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
