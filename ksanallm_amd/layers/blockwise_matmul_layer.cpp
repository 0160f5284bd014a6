#include "blockwise_matmul_layer.h"

namespace ksana_llm {

static inline size_t DivRoundUpSz(size_t a, size_t b) { return (a + b - 1) / b; }

Status BlockwiseMatMulLayer::Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
                                  std::shared_ptr<Context> context, int rank) {
  STATUS_CHECK_FAILURE(BaseLayer::Init(parameters, runtime_config, context, rank));
  if (parameters.size() < 5) return Status(RET_INVALID_ARGUMENT, "BlockwiseMatMulLayer: expects >= 5 init parameters");
  size_t parameter_index = 0;
  max_m_ = std::any_cast<size_t>(parameters[parameter_index++]);
  n_ = std::any_cast<size_t>(parameters[parameter_index++]);
  k_ = std::any_cast<size_t>(parameters[parameter_index++]);
  block_size_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  weight_ = std::any_cast<Tensor>(parameters[parameter_index++]);
  if (parameter_index < parameters.size()) {
    skip_quant_ = std::any_cast<const bool>(parameters[parameter_index++]);
  }
  if (block_size_ != 128) return Status(RET_INVALID_ARGUMENT, "BlockwiseMatMulLayer: block size must be 128");
  return Status();
}

size_t BlockwiseMatMulLayer::GetWorkspaceSize() {
  const size_t input_size = max_m_ * k_ * GetTypeSize(TYPE_FP8_E4M3);
  const size_t scale_size = max_m_ * DivRoundUpSz(k_, block_size_) * GetTypeSize(TYPE_FP32);
  // the GEMM's scratch starts behind the quantized activations on a 256-byte boundary (the library asks for 16-byte
  // alignment, and max_m * k/128 floats is a multiple of 16 bytes only for some max_m)
  input_buffer_size_ = (input_size + scale_size + 255) / 256 * 256;
  gemm_workspace_size_ = ksq_fp8_blockwise_workspace_size(max_m_, n_, k_);
  workspace_size_ = input_buffer_size_ + gemm_workspace_size_;
  return workspace_size_;
}

Status BlockwiseMatMulLayer::Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) {
  ksq_tile_desc desc;
  const int dtype = KsqDtypeOrFp32(inter_data_type_, "BlockwiseMatMulLayer");
  if (ksq_select_tile(KSQ_KIND_FP8_BLOCKWISE, max_m_ ? max_m_ : 1, n_, k_, dtype == KSQ_F32 ? KSQ_BF16 : dtype, &desc) != KSQ_OK) {
    return Status(RET_INVALID_ARGUMENT, std::string("BlockwiseMatMulLayer: ") + ksq_last_error_string());
  }
  return Status();
}

Status BlockwiseMatMulLayer::Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) {
  if (!workspace_buffer_ || workspace_size_ > workspace_buffer_->GetTotalBytes()) {
    KLLM_THROW("workspace size " + std::to_string(workspace_size_) + " > buffer size " +
               std::to_string(workspace_buffer_ ? workspace_buffer_->GetTotalBytes() : 0));
  }
  const size_t m = input_tensors[0].shape[0];
  const size_t k = input_tensors[0].shape[1];
  if (k != k_ && k != 2 * k_) KLLM_THROW("BlockwiseMatMulLayer: activation inner dimension must be k or 2k");
  if (m > max_m_) KLLM_THROW("BlockwiseMatMulLayer: m exceeds max_m");
  if (!input_tensors[1].weight_scales) KLLM_THROW("BlockwiseMatMulLayer: weight tensor has no weight_scales bound");
  const int dtype = KsqDtypeOrFp32(inter_data_type_, "BlockwiseMatMulLayer");  // fp32: DISPATCH_BY_3_DTYPE of the reference's Forward
  hipStream_t stream = context_->GetComputeStreams()[rank_].Get();

  char* base = workspace_buffer_->GetPtr<char>();
  void* a_q = base;
  void* a_s = base + GetTypeSize(TYPE_FP8_E4M3) * m * k_;
  if (!skip_quant_) {
    KsqCheck(ksq_fp8_group_quant(input_tensors[0].GetPtr<void>(), a_q, a_s, m, k_, block_size_, /*column_major*/ 1,
                                 /*fuse_silu_mul*/ k == 2 * k_ ? 1 : 0, dtype, stream),
             "BlockwiseMatMulLayer");
  }
  void* b = input_tensors[1].GetPtr<void>();
  void* b_s = input_tensors[1].weight_scales->GetPtr<void>();
  KsqCheck(ksq_fp8_blockwise_gemm(a_q, a_s, b, b_s, output_tensors[0].GetPtr<void>(), m, n_, k_, dtype,
                                  base + input_buffer_size_, gemm_workspace_size_, stream),
           "BlockwiseMatMulLayer");
  output_tensors[0].shape = {m, n_};
  output_tensors[0].dtype = input_tensors[0].dtype;
  return Status();
}

}  // namespace ksana_llm
