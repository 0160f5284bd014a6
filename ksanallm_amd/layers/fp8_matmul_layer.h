// Per-tensor FP8 (e4m3) matmul layer: one fp32 scale for the weight, one for the activations.
// Mirrors src/ksana_llm/layers/fp8_matmul_layer.h:13 and nvidia/fp8_matmul_layer.cpp:13-100: the activations are
// quantized into the workspace (dynamically, or with the checkpoint's static input_scales when the weight tensor has
// them bound) and multiplied with the [n, k] e4m3 weight.  The reference hands the product to cuBLASLt with scale
// pointers and looks up a tuned algorithm; here the blockwise MFMA kernels do the work with both scales spread into
// their layouts, so there is nothing to look up.
#pragma once

#include "base_layer.h"

namespace ksana_llm {

class Fp8MatMulLayer : public BaseLayer {
 public:
  // parameters: size_t max_m, size_t max_k
  Status Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
              std::shared_ptr<Context> context, int rank) override;
  // bytes for m x k activations: quantized codes + one scale + the GEMM's own scratch (a fixed budget, as the
  // reference's cuBLAS workspace is: n is not known before Forward)
  size_t GetWorkspaceSize(const int m, const int k);
  size_t GetWorkspaceSize() override;
  // inputs: [0] activations [m, k] T, [1] weight [n, k] e4m3 packed by PackFp8Weight (quant_weight_repack.h), with
  // weight_scales (1 fp32) and optionally input_scales
  // (1 fp32, static activation scale).  output [0]: [m, n] in T.
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;

  // scratch of the GEMM: the partial tiles of a split along K (at most 512 tiles of 256 x 256 fp32) and the spread scales
  static constexpr size_t kGemmWorkspaceBytes = (size_t(512) * 256 * 256 * 4) + (size_t(8) << 20);

 private:
  size_t max_m_ = 0;
  size_t max_k_ = 0;
};

}  // namespace ksana_llm
