// GPTQ / AWQ int4 group-wise matmul layers.  The reference has three classes, one per NVIDIA kernel family; on MI355X
// one kernel library serves all of them, so the three names are thin subclasses of one implementation that keep the
// reference's Init parameter order and its per-class restrictions where they are part of the contract.
//   CutlassMatMulLayer   src/ksana_llm/layers/cutlass_matmul_layer.h:25, nvidia/cutlass_matmul_layer.cpp:37-182
//   MarlinMatMulLayer    src/ksana_llm/layers/marlin_matmul_layer.h:23, nvidia/marlin_matmul_layer.cpp:12-96
//   MacheteMatMulLayer   src/ksana_llm/layers/machete_matmul_layer.h:23, nvidia/machete_matmul_layer.cpp
//
// Forward inputs: [0] activations [m, k] in T, [1] the weight in the CDNA4 packed layout with `scales` (and, for AWQ,
// `zeros`) bound to it by PackGroupQuantWeight() (quant_weight_repack.h).  Output [0] is [m, n] in T.
// GPTQ act-order (is_gptq_desc): the packed rows are sorted by quantization group and the weight carries `perm`; the
// layer gathers the activation columns through it into its workspace in front of the GEMM (the reference's Marlin
// kernel does the same gather internally).
#pragma once

#include "base_layer.h"

namespace ksana_llm {

class W4A16MatMulLayer : public BaseLayer {
 public:
  // parameters: size_t max_m, size_t max_n, size_t max_k, size_t groupsize, bool is_awq, bool is_gptq_desc,
  //             bool is_k_full, bool cutlass_use_gemv_cuda_core, DataType weight_data_type
  Status Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
              std::shared_ptr<Context> context, int rank) override;
  size_t GetWorkspaceSize() override;
  // The reference times every tactic for m = 1..max_batch here; tile choice is a closed-form function of the shape
  // on this hardware (ksq_select_tile), so this only validates that a kernel exists for the layer's shape.
  Status Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) override;
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;

 protected:
  virtual const char* Name() const { return "W4A16MatMulLayer"; }

  DataType weight_data_type_ = TYPE_INVALID;
  bool is_awq_ = false;
  bool is_gptq_desc_ = false;
  bool is_k_full_ = true;
  size_t max_m_ = 0, max_n_ = 0, max_k_ = 0;
  size_t groupsize_ = 0;
  size_t tp_cut_bound_ = 1;  // the largest tensor-parallel size the runtime configuration names
  size_t workspace_size_ = 0;
  size_t gemm_workspace_size_ = 0, permuted_input_size_ = 0;
};

class CutlassMatMulLayer : public W4A16MatMulLayer {
 protected:
  const char* Name() const override { return "CutlassMatMulLayer"; }
};

class MarlinMatMulLayer : public W4A16MatMulLayer {
 protected:
  const char* Name() const override { return "MarlinMatMulLayer"; }
};

class MacheteMatMulLayer : public W4A16MatMulLayer {
 protected:
  const char* Name() const override { return "MacheteMatMulLayer"; }
};

}  // namespace ksana_llm
