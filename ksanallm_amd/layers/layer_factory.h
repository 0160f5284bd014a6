// Factories keyed like the reference's: (weight type, input type, output type, quant mode, backend) -> layer class.
//   MatMulLayerFactory  src/ksana_llm/layers/matmul_layer_factory.h:24, matmul_layer_factory.cpp:20-245
//   MoeLayerFactory     src/ksana_llm/layers/moe_layer_factory.h, moe_layer_factory.cpp:22-75
// Only the quantized rows are registered: unquantized layers stay with the host framework.  Every backend name the
// reference accepts for int4 weights (cutlass / marlin / machete) resolves to a layer here, so a model config that
// names any of them keeps working.
#pragma once

#include <map>
#include <tuple>

#include "base_layer.h"

namespace ksana_llm {

class MatMulLayerFactory {
 public:
  typedef std::shared_ptr<BaseLayer> (MatMulLayerFactory::*BuildLayerFunc)();
  MatMulLayerFactory(const ModelConfig& model_config, const RuntimeConfig& runtime_config, const int rank,
                     std::shared_ptr<Context> context);

  template <typename ClassT>
  std::shared_ptr<BaseLayer> BuildLayer() {
    return std::make_shared<ClassT>();
  }

  // Throws (KLLM_THROW) for a combination with no registered layer, like the reference.
  std::shared_ptr<BaseLayer> CreateLayer(DataType weight_type, DataType input_type, DataType output_type,
                                         const std::vector<std::any>& init_params, QuantMode quant_mode,
                                         LinearComputeBackend backend);

  // The group-quant parameter vector AutoCreateLayer builds for a dense GPTQ / AWQ projection
  // (matmul_layer_factory.cpp:160-169): m, n, k, groupsize, awq, gptq desc, k full, cuda gemv, weight data type.
  std::vector<std::any> GroupMatMulParams(size_t n, size_t k, bool k_full) const;

 private:
  std::shared_ptr<Context> context_;
  int rank_;
  ModelConfig model_config_;
  RuntimeConfig runtime_config_;
  std::map<std::tuple<DataType, DataType, DataType, QuantMode, LinearComputeBackend>, BuildLayerFunc> builder_map_;
};

class MoeLayerFactory {
 public:
  typedef std::shared_ptr<BaseLayer> (MoeLayerFactory::*BuildLayerFunc)();
  MoeLayerFactory(const ModelConfig& model_config, const RuntimeConfig& runtime_config, const int rank,
                  std::shared_ptr<Context> context);

  template <typename ClassT>
  std::shared_ptr<BaseLayer> BuildLayer() {
    return std::make_shared<ClassT>();
  }

  std::shared_ptr<BaseLayer> CreateLayer(DataType weight_type, DataType input_type, DataType output_type,
                                         const std::vector<std::any>& init_params, QuantMode quant_mode,
                                         MoeComputeBackend backend);

 private:
  std::shared_ptr<Context> context_;
  int rank_;
  ModelConfig model_config_;
  RuntimeConfig runtime_config_;
  std::map<std::tuple<DataType, DataType, DataType, QuantMode, MoeComputeBackend>, BuildLayerFunc> builder_map_;
};

}  // namespace ksana_llm
