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

  // The call model code makes (modules/basic/linear.cpp:24-33): decides the layer class and assembles its init
  // parameters from the weight's name, the loader's record of it and the model configuration
  // (matmul_layer_factory.cpp:87-217).  Only the quantized branches exist here: a weight that is none of W4A8, GPTQ / AWQ
  // group-quantized or fp8 throws, where the reference falls through to its unquantized MatMulLayer.
  std::shared_ptr<BaseLayer> AutoCreateLayer(std::shared_ptr<BaseWeight> base_weight, std::string weight_name,
                                             DataType weight_type, DataType input_type, DataType output_type,
                                             LinearComputeBackend backend, const std::vector<std::any>& init_params);

  // The group-quant parameter vector AutoCreateLayer builds for a dense GPTQ / AWQ projection
  // (matmul_layer_factory.cpp:160-169): m, n, k, groupsize, awq, gptq desc, k full, cuda gemv, weight data type.
  std::vector<std::any> GroupMatMulParams(size_t n, size_t k, bool k_full) const;

  // (k, n, k_full) of the projection whose name occurs in weight_name, per GPU, computed from the model configuration
  // because the packed layouts no longer show them (matmul_layer_factory.cpp:106-157).  k_full is false for the
  // row-parallel projections, whose K is cut over the tensor-parallel ranks.  False when no projection matches.
  bool ProjectionShape(const std::string& weight_name, size_t* k, size_t* n, bool* k_full) const;

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

  // The call model code makes for the expert block (moe_layer_factory.cpp:77-193): weight_names = {up_gate experts,
  // down experts}, init_params = {MoeScaleNormMode}.  Checks the two stacks against each other, decides between int4
  // (GPTQ experts, also as a sub-configuration of an fp8 model), block-fp8 and neither, and appends the 20 further init
  // parameters in the order MoeLayer::Init reads them.  Expert weights this library has no layer for throw.
  std::shared_ptr<BaseLayer> AutoCreateMoeLayer(std::shared_ptr<BaseWeight> base_weight,
                                                std::vector<std::string> weight_names, DataType weight_type,
                                                DataType input_type, DataType output_type, int layer_idx,
                                                const std::vector<std::any>& init_params);

 private:
  std::shared_ptr<Context> context_;
  int rank_;
  ModelConfig model_config_;
  RuntimeConfig runtime_config_;
  std::map<std::tuple<DataType, DataType, DataType, QuantMode, MoeComputeBackend>, BuildLayerFunc> builder_map_;
};

}  // namespace ksana_llm
