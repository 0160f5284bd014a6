// Blockwise-FP8 (e4m3, 128x128 weight scales) matmul layer.
// Mirrors src/ksana_llm/layers/blockwise_matmul_layer.h:15 and nvidia/blockwise_matmul_layer.cpp:16-299:
// activations are quantized per token / per 128 channels into the head of the workspace (a_q at offset 0, a_s right
// after the cur_m*k quantized bytes, column-major), then multiplied with the weight, which the loader has put into the
// packed fragment layout (PackFp8Weight, quant_weight_repack.h).
// The reference picks between Cutlass / DeepGEMM / DeepGEMM-swapAB by timing them in Preprocess; here the variant is a
// pure function of (m, n, k), so Preprocess has nothing to search and the m -> RoundUp(m, 4) padding DeepGEMM needs
// does not exist.
#pragma once

#include "base_layer.h"

namespace ksana_llm {

class BlockwiseMatMulLayer : public BaseLayer {
 public:
  // parameters: size_t max_m, size_t n, size_t k, size_t block_size, Tensor weight [, bool skip_quant]
  Status Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
              std::shared_ptr<Context> context, int rank) override;
  size_t GetWorkspaceSize() override;
  Status Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) override;
  // inputs: [0] activations [m, k] (or [m, 2k]: silu(x[:, :k]) * x[:, k:] is fused into the quantizer),
  //         [1] weight [n, k] e4m3 packed by PackFp8Weight, with weight_scales [ceil(n/128), k/128] fp32.
  // output [0]: [m, n] in T.
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;

 private:
  size_t max_m_ = 0;
  size_t n_ = 0;
  size_t k_ = 0;
  size_t block_size_ = 128;
  Tensor weight_;
  size_t workspace_size_ = 0;
  size_t input_buffer_size_ = 0;
  size_t gemm_workspace_size_ = 0;
  // quantization has already been performed elsewhere and stored in the workspace buffer
  bool skip_quant_ = false;
};

}  // namespace ksana_llm
