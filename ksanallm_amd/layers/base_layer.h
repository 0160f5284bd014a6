// Layer interface the model code drives: Init -> GetWorkspaceSize -> SetWorkspaceBuffer -> Preprocess -> Forward.
// Same virtuals, defaults and protected members as src/ksana_llm/layers/base_layer.h:45-91.
#pragma once

#include "ksana_compat.h"
#include "ksq.h"

#ifdef KSQ_IN_KSANA_TREE
#  include "ksana_llm/layers/base_layer.h"
#else
namespace ksana_llm {

class BaseLayer {
 public:
  virtual ~BaseLayer() = default;

  virtual Status Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
                      std::shared_ptr<Context> context, int rank) {
    context_ = context;
    rank_ = rank;
    inter_data_type_ = runtime_config.inter_data_type;
    tp_size_ = context_->GetTensorParallelSize();
    dp_size_ = static_cast<int>(runtime_config.parallel_basic_config.attn_data_parallel_size);
    attn_dp_atp_size_ = static_cast<int>(runtime_config.parallel_basic_config.attn_tensor_parallel_size);
    if (attn_dp_atp_size_ == 0) attn_dp_atp_size_ = 1;
    attn_dp_group_id_ = rank_ / attn_dp_atp_size_;
    attn_dp_rank_id_ = rank_ % attn_dp_atp_size_;
    return Status();
  }

  virtual size_t GetWorkspaceSize() { return 0; }

  virtual Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) = 0;

  virtual Status SetWorkspaceBuffer(const std::shared_ptr<Tensor>& workspace_buffer) {
    workspace_buffer_ = workspace_buffer;
    return Status();
  }

  virtual Status Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) { return Status(); }

  virtual void Clear() {}

 protected:
  DataType inter_data_type_ = TYPE_FP16;
  int rank_ = 0;
  std::shared_ptr<Context> context_;
  std::shared_ptr<Tensor> workspace_buffer_;
  int tp_size_ = 1;
  int dp_size_ = 1;
  int attn_dp_atp_size_ = 1;
  int attn_dp_group_id_ = 0;
  int attn_dp_rank_id_ = 0;
};

}  // namespace ksana_llm
#endif

namespace ksana_llm {

// activation type of the reference's template parameter T -> tag of the kernel library; fp32 activations are taken by
// the fp8 layers only (KsqDtypeOrFp32), the int4 kernels multiply 16-bit activations
inline int KsqDtype(DataType dtype, const char* who) {
  if (dtype == TYPE_FP16) return KSQ_F16;
  if (dtype == TYPE_BF16) return KSQ_BF16;
  KLLM_THROW(std::string(who) + ": Unsupported Dtype type: " + std::to_string(static_cast<int>(dtype)));
}

// the same for the layers whose kernels also take fp32 activations (the block-fp8 quantizer and GEMM, which the
// reference instantiates for float: basic_kernel_wrapper.cpp:1096,1237)
inline int KsqDtypeOrFp32(DataType dtype, const char* who) {
  return dtype == TYPE_FP32 ? KSQ_F32 : KsqDtype(dtype, who);
}

// kernel-library status -> exception, like KLLM_KERNEL_CHECK does for a failed launch
inline void KsqCheck(int rc, const char* who) {
  if (rc != KSQ_OK) KLLM_THROW(std::string(who) + ": " + ksq_last_error_string());
}

}  // namespace ksana_llm
