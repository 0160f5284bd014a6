#include "w4a16_matmul_layer.h"

#include <algorithm>

namespace ksana_llm {

Status W4A16MatMulLayer::Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
                              std::shared_ptr<Context> context, int rank) {
  STATUS_CHECK_FAILURE(BaseLayer::Init(parameters, runtime_config, context, rank));
  if (parameters.size() < 9) {
    return Status(RET_INVALID_ARGUMENT, std::string(Name()) + ": expects 9 init parameters");
  }
  int parameter_index = 0;
  max_m_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  max_n_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  max_k_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  groupsize_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  is_awq_ = std::any_cast<const bool>(parameters[parameter_index++]);
  is_gptq_desc_ = std::any_cast<const bool>(parameters[parameter_index++]);
  is_k_full_ = std::any_cast<const bool>(parameters[parameter_index++]);
  [[maybe_unused]] bool use_gemv_cuda_core = std::any_cast<const bool>(parameters[parameter_index++]);  // no analogue
  weight_data_type_ = std::any_cast<const DataType>(parameters[parameter_index++]);
  is_k_full_ = is_gptq_desc_ ? is_k_full_ : true;
  tp_cut_bound_ = std::max({runtime_config.parallel_basic_config.tensor_parallel_size,
                            runtime_config.parallel_basic_config.attn_tensor_parallel_size,
                            runtime_config.parallel_basic_config.moe_tensor_para_size});
  if (is_gptq_desc_ && is_awq_) return Status(RET_INVALID_ARGUMENT, std::string(Name()) + ": desc_act belongs to GPTQ, not AWQ");
  return Status();
}

size_t W4A16MatMulLayer::GetWorkspaceSize() {
  if (weight_data_type_ != TYPE_I4_GROUP) {
    KLLM_THROW(std::string("Not supported weight data type: ") + std::to_string(weight_data_type_) + ". " + Name() +
               " only supports TYPE_I4_GROUP.");
  }
  gemm_workspace_size_ = ksq_w4a16_workspace_size(max_m_, max_n_, max_k_, groupsize_, KsqDtype(inter_data_type_, Name()));
  gemm_workspace_size_ = (gemm_workspace_size_ + 255) & ~static_cast<size_t>(255);
  // act-order: the activations with their columns permuted, behind the GEMM's scratch
  // (a K range of an act-order weight is packed with every run of equal group padded to 32 rows: up to 31 more rows
  // for each of the checkpoint's groups - k * ranks / groupsize of them - that has rows in the range)
  size_t permuted_k = max_k_;
  if (is_gptq_desc_ && !is_k_full_) {
    // the cut the factory applied is one of the tensor-parallel sizes the configuration names (o_proj and the MLA
    // projections are cut by the attention size, the MLP by the general one): the largest of them bounds the groups
    const size_t ranks = std::max<size_t>({static_cast<size_t>(std::max(1, context_->GetTensorParallelSize())), tp_cut_bound_, 1});
    const size_t groups = std::min(max_k_, max_k_ * ranks / std::max<size_t>(1, groupsize_));
    permuted_k = (max_k_ + 31 * groups + 127) / 128 * 128;
    // the GEMM then runs over the padded rows with group size 32: its scratch for any padded depth up to the bound
    const int dtype = KsqDtype(inter_data_type_, Name());
    for (size_t kk = (max_k_ + 127) / 128 * 128; kk <= permuted_k; kk += 128) {
      const size_t need = (ksq_w4a16_workspace_size(max_m_, max_n_, kk, 32, dtype) + 255) & ~static_cast<size_t>(255);
      gemm_workspace_size_ = std::max(gemm_workspace_size_, need);
    }
  }
  permuted_input_size_ = is_gptq_desc_ ? max_m_ * permuted_k * GetTypeSize(inter_data_type_) : 0;
  workspace_size_ = gemm_workspace_size_ + permuted_input_size_;
  return workspace_size_;
}

Status W4A16MatMulLayer::Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) {
  ksq_tile_desc desc;
  const int dtype = KsqDtype(inter_data_type_, Name());
  const size_t probe_m[2] = {1, max_m_ ? max_m_ : 1};
  for (size_t m : probe_m) {
    if (ksq_select_tile(KSQ_KIND_W4A16, m, max_n_, max_k_, dtype, &desc) != KSQ_OK) {
      return Status(RET_INVALID_ARGUMENT, std::string(Name()) + ": " + ksq_last_error_string());
    }
  }
  return Status();
}

Status W4A16MatMulLayer::Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) {
  if (weight_data_type_ != TYPE_I4_GROUP) {
    KLLM_THROW(std::string("Not supported weight data type: ") + std::to_string(weight_data_type_) + ". " + Name() +
               " only supports TYPE_I4_GROUP.");
  }
  const Tensor& weight_tensor = input_tensors[1];
  if (!weight_tensor.scales) KLLM_THROW(std::string(Name()) + ": weight tensor has no scales bound");
  if (is_awq_ && !weight_tensor.zeros) KLLM_THROW(std::string(Name()) + ": AWQ weight tensor has no zeros bound");
  void* p_qweight = weight_tensor.GetPtr<void>();
  void* p_scales = weight_tensor.scales->GetPtr<void>();
  void* p_zeros = is_awq_ ? weight_tensor.zeros->GetPtr<void>() : nullptr;

  const size_t m = input_tensors[0].shape[0];
  const size_t n = max_n_;
  const size_t k = max_k_;
  if (input_tensors[0].shape.size() < 2 || input_tensors[0].shape[1] != k) {
    KLLM_THROW(std::string(Name()) + ": activation inner dimension does not match k");
  }
  char* ws = workspace_buffer_ ? workspace_buffer_->GetPtr<char>() : nullptr;
  size_t ws_bytes = workspace_buffer_ ? workspace_buffer_->GetTotalBytes() : 0;
  const void* x = input_tensors[0].GetPtr<void>();
  const int dtype = KsqDtype(inter_data_type_, Name());
  hipStream_t stream = context_->GetComputeStreams()[rank_].Get();
  if (is_gptq_desc_) {
    // rows of the packed weight are sorted by quantization group (perm): read the activation columns the same way
    if (!weight_tensor.perm) KLLM_THROW(std::string(Name()) + ": act-order weight tensor has no perm bound");
    if (m > max_m_) KLLM_THROW(std::string(Name()) + ": m exceeds max_m");
    if (!ws || ws_bytes < gemm_workspace_size_ + m * k * GetTypeSize(inter_data_type_)) {
      KLLM_THROW(std::string(Name()) + ": workspace buffer missing or smaller than GetWorkspaceSize()");
    }
    void* permuted = ws + gemm_workspace_size_;
    if (!is_k_full_) {
      // a K range of the checkpoint, packed with padded runs of equal group (PackGroupQuantWeight, k_full = false):
      // K' packed rows, one scale row per 32 of them
      const size_t kp = weight_tensor.shape.empty() ? 0 : weight_tensor.shape[0];
      if (kp < k || kp % 128 != 0 || weight_tensor.perm->GetElementNumber() != kp ||
          weight_tensor.scales->shape.empty() || weight_tensor.scales->shape[0] * 32 != kp) {
        KLLM_THROW(std::string(Name()) + ": act-order weight cut along K must come from PackGroupQuantWeight with k_full = false");
      }
      if (ws_bytes < gemm_workspace_size_ + m * kp * GetTypeSize(inter_data_type_)) {
        KLLM_THROW(std::string(Name()) + ": workspace buffer smaller than the padded activations need");
      }
      KsqCheck(ksq_gather_columns(x, weight_tensor.perm->GetPtr<void>(), permuted, m, k, kp, dtype, stream), Name());
      KsqCheck(ksq_w4a16_gemm(output_tensors[0].GetPtr<void>(), permuted, p_qweight, p_scales, nullptr, ws, gemm_workspace_size_,
                              m, n, kp, 32, dtype, stream),
               Name());
      output_tensors[0].shape = {m, n};
      output_tensors[0].dtype = input_tensors[0].dtype;
      return Status();
    }
    KsqCheck(ksq_permute_columns(x, weight_tensor.perm->GetPtr<void>(), permuted, m, k, dtype, stream), Name());
    x = permuted;
    ws_bytes = gemm_workspace_size_;
  }
  KsqCheck(ksq_w4a16_gemm(output_tensors[0].GetPtr<void>(), x, p_qweight, p_scales, p_zeros, ws, ws_bytes, m, n, k,
                          groupsize_, dtype, stream),
           Name());
  output_tensors[0].shape = {m, n};
  output_tensors[0].dtype = input_tensors[0].dtype;
  return Status();
}

}  // namespace ksana_llm
