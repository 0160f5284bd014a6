#include "finegrained_mixed_dtype_gemm_layer.h"

namespace ksana_llm {

static inline size_t AlignTo256(size_t size) { return (size + 255) & ~static_cast<size_t>(255); }

Status FinegrainedMixedDtypeGemmLayer::Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
                                            std::shared_ptr<Context> context, int rank) {
  STATUS_CHECK_FAILURE(BaseLayer::Init(parameters, runtime_config, context, rank));
  if (parameters.empty()) return Status(RET_INVALID_ARGUMENT, "FinegrainedMixedDtypeGemmLayer: expects its parameter struct");
  params_ = std::any_cast<const FinegrainedMixedDtypeGemmLayerParameters>(parameters.front());
  if (params_.group_size != 128 && params_.group_size != 64) {
    return Status(RET_INVALID_ARGUMENT, "FinegrainedMixedDtypeGemmLayer: group size " + std::to_string(params_.group_size) +
                                            " has no kernel (128 or 64)");
  }
  if (params_.has_zero) return Status(RET_INVALID_ARGUMENT, "FinegrainedMixedDtypeGemmLayer: zero points have no kernel");
  if (params_.activation_type != TYPE_FP8_E4M3) {
    return Status(RET_INVALID_ARGUMENT, "FinegrainedMixedDtypeGemmLayer: activation type must be TYPE_FP8_E4M3");
  }
  if (params_.output_type != TYPE_FP16 && params_.output_type != TYPE_BF16) {
    return Status(RET_INVALID_ARGUMENT, "FinegrainedMixedDtypeGemmLayer: output type must be fp16 or bf16");
  }
  if (params_.n == 0 || params_.k == 0 || params_.n % 16 != 0 || params_.k % 128 != 0) {
    return Status(RET_INVALID_ARGUMENT, "FinegrainedMixedDtypeGemmLayer: n must be a multiple of 16 and k of 128");
  }
  return Status();
}

size_t FinegrainedMixedDtypeGemmLayer::GetWorkspaceSize() {
  kernel_workspace_size_ = AlignTo256(ksq_w4a8_workspace_size(params_.m, params_.n, params_.k));
  quantized_size_ = AlignTo256(params_.m * params_.k * sizeof(char));
  sums_size_ = AlignTo256(params_.m * (params_.k / params_.group_size) * sizeof(float));
  return kernel_workspace_size_ + quantized_size_ + sums_size_;
}

Status FinegrainedMixedDtypeGemmLayer::Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) {
  (void)model_config;
  (void)runtime_config;
  return Status();
}

Status FinegrainedMixedDtypeGemmLayer::Forward(const std::vector<Tensor>& input_tensors,
                                               std::vector<Tensor>& output_tensors) {
  const size_t m = input_tensors[0].shape[0];
  const size_t n = 2 * input_tensors[1].shape[1];
  const size_t k = input_tensors[0].shape[1];
  if (input_tensors[1].shape[0] != k || n != params_.n || k != params_.k) {
    KLLM_THROW("FinegrainedMixedDtypeGemmLayer: weight must be [k, n/2] with the n and k given to Init");
  }
  if (m > params_.m) KLLM_THROW("FinegrainedMixedDtypeGemmLayer: more tokens than the m given to Init");
  const size_t need = GetWorkspaceSize();
  if (!workspace_buffer_ || need > workspace_buffer_->GetTotalBytes()) {
    KLLM_THROW("workspace size " + std::to_string(need) + " > buffer size " +
               std::to_string(workspace_buffer_ ? workspace_buffer_->GetTotalBytes() : 0));
  }
  const Tensor& weight = input_tensors[1];
  if (!weight.weight_scales || weight.weight_scales->GetPtr<void>() == nullptr) {
    KLLM_THROW("Cannot load weight_scale. Weight_scale is nullptr.");
  }
  if (!weight.pre_quant_scales && (!weight.input_scales || weight.input_scales->GetPtr<void>() == nullptr)) {
    KLLM_THROW("FinegrainedMixedDtypeGemmLayer: the weight carries neither input_scales nor pre_quant_scales");
  }
  const int dtype = KsqDtype(input_tensors[0].dtype, "FinegrainedMixedDtypeGemmLayer");
  const int out_dtype = KsqDtype(params_.output_type, "FinegrainedMixedDtypeGemmLayer");
  hipStream_t stream = context_->GetComputeStreams()[rank_].Get();

  char* kernel_workspace = workspace_buffer_->GetPtr<char>();
  char* quantized_input = kernel_workspace + kernel_workspace_size_;
  char* group_sums = quantized_input + quantized_size_;
  const int sums = params_.group_size == 64 ? KSQ_W4A8_SUMS_PER_64 : 0;  // one activation sum per scale group
  if (weight.pre_quant_scales) {
    KsqCheck(ksq_w4a8_static_quant(input_tensors[0].GetPtr<void>(), weight.pre_quant_scales->GetPtr<void>(), quantized_input,
                                   group_sums, m, k, KSQ_W4A8_PER_CHANNEL | sums, dtype, stream),
             "FinegrainedMixedDtypeGemmLayer");
  } else {
    KsqCheck(ksq_w4a8_static_quant(input_tensors[0].GetPtr<void>(), weight.input_scales->GetPtr<void>(), quantized_input,
                                   group_sums, m, k, KSQ_W4A8_PER_TENSOR | sums, dtype, stream),
             "FinegrainedMixedDtypeGemmLayer");
  }
  KsqCheck(ksq_w4a8_gemm(quantized_input, group_sums, weight.GetPtr<void>(), weight.weight_scales->GetPtr<void>(),
                         weight.alpha, output_tensors[0].GetPtr<void>(), m, n, k, params_.group_size, out_dtype,
                         kernel_workspace, kernel_workspace_size_, stream),
           "FinegrainedMixedDtypeGemmLayer");
  output_tensors[0].shape = {m, n};
  output_tensors[0].dtype = input_tensors[0].dtype;
  return Status();
}

}  // namespace ksana_llm
