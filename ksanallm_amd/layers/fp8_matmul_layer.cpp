#include "fp8_matmul_layer.h"

namespace ksana_llm {

static inline size_t Align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

Status Fp8MatMulLayer::Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
                            std::shared_ptr<Context> context, int rank) {
  STATUS_CHECK_FAILURE(BaseLayer::Init(parameters, runtime_config, context, rank));
  if (parameters.size() < 2) return Status(RET_INVALID_ARGUMENT, "Fp8MatMulLayer: expects max_m, max_k");
  int parameter_index = 0;
  max_m_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  max_k_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  if (max_k_ % 128 != 0) return Status(RET_INVALID_ARGUMENT, "Fp8MatMulLayer: k must be a multiple of 128");
  KsqDtypeOrFp32(inter_data_type_, "Fp8MatMulLayer");
  return Status();
}

size_t Fp8MatMulLayer::GetWorkspaceSize(const int m, const int k) {
  // [GEMM scratch][m*k quantized activations][one fp32 scale], the order of the reference's buffer
  const size_t input_size = Align256(static_cast<size_t>(m) * k * GetTypeSize(TYPE_FP8_E4M3));
  return kGemmWorkspaceBytes + input_size + Align256(GetTypeSize(TYPE_FP32));
}

size_t Fp8MatMulLayer::GetWorkspaceSize() { return GetWorkspaceSize(static_cast<int>(max_m_), static_cast<int>(max_k_)); }

Status Fp8MatMulLayer::Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) {
  const size_t m = input_tensors[0].shape[0];
  const size_t k = input_tensors[0].shape[1];
  const size_t n = input_tensors[1].shape[0];
  const size_t workspace_size = GetWorkspaceSize(static_cast<int>(m), static_cast<int>(k));
  if (!workspace_buffer_ || workspace_size > workspace_buffer_->GetTotalBytes()) {
    KLLM_THROW("workspace size " + std::to_string(workspace_size) + " > buffer size " +
               std::to_string(workspace_buffer_ ? workspace_buffer_->GetTotalBytes() : 0));
  }
  if (!input_tensors[1].weight_scales || input_tensors[1].weight_scales->GetPtr<void>() == nullptr) {
    KLLM_THROW("Cannot load weight_scale. Weight_scale is nullptr.");
  }
  if (input_tensors[1].shape.size() < 2 || input_tensors[1].shape[1] != k) KLLM_THROW("Fp8MatMulLayer: weight must be [n, k]");
  const size_t gemm_need = ksq_fp8_tensor_gemm_workspace_size(m, n, k);
  if (gemm_need > kGemmWorkspaceBytes) {
    KLLM_THROW("Fp8MatMulLayer: GEMM scratch " + std::to_string(gemm_need) + " exceeds the budget " +
               std::to_string(kGemmWorkspaceBytes));
  }
  const int dtype = KsqDtypeOrFp32(inter_data_type_, "Fp8MatMulLayer");
  hipStream_t stream = context_->GetComputeStreams()[rank_].Get();

  char* gemm_workspace = workspace_buffer_->GetPtr<char>();
  char* input_quant = gemm_workspace + kGemmWorkspaceBytes;
  const void* weight_quant = input_tensors[1].GetPtr<void>();
  const void* weight_scale = input_tensors[1].weight_scales->GetPtr<void>();
  float* input_scale = nullptr;
  if (input_tensors[1].input_scales) {  // static: the checkpoint's activation scale
    input_scale = input_tensors[1].input_scales->GetPtr<float>();
    KsqCheck(ksq_fp8_channel_quant(input_tensors[0].GetPtr<void>(), input_quant, input_scale, 1, m * k, 1, dtype, stream),
             "Fp8MatMulLayer");
  } else {
    input_scale = reinterpret_cast<float*>(input_quant + Align256(GetTypeSize(TYPE_FP8_E4M3) * m * k));
    KsqCheck(ksq_fp8_channel_quant(input_tensors[0].GetPtr<void>(), input_quant, input_scale, 1, m * k, 0, dtype, stream),
             "Fp8MatMulLayer");
  }
  KsqCheck(ksq_fp8_tensor_gemm(input_quant, input_scale, weight_quant, weight_scale, output_tensors[0].GetPtr<void>(), m, n,
                               k, dtype, gemm_workspace, kGemmWorkspaceBytes, stream),
           "Fp8MatMulLayer");
  output_tensors[0].shape = {m, n};
  output_tensors[0].dtype = input_tensors[0].dtype;
  return Status();
}

}  // namespace ksana_llm
