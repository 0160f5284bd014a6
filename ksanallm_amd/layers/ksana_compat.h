// Stand-ins for the handful of KsanaLLM framework types the quantized layers touch, so that the layer classes in this
// directory build and run on their own.  Inside the KsanaLLM tree define KSQ_IN_KSANA_TREE: the real headers are used
// and nothing below is compiled.
//
// Every type keeps the member names, enumerator order and call signatures of its counterpart:
//   Status/RetCode          src/ksana_llm/utils/status.h, ret_code.h
//   DataType, GetTypeSize   src/ksana_llm/utils/device_types.h:44-90
//   Tensor                  src/ksana_llm/utils/tensor.h (shape/dtype/GetPtr and the quantization side tensors)
//   Context, Stream         src/ksana_llm/utils/context.h, utils/nvidia/cuda_utils.h
//   RuntimeConfig           src/ksana_llm/utils/config/schedule_config_parser.h:316
//   ModelConfig, QuantConfig, MoeConfig, MlaConfig, QuantMode, LinearComputeBackend, MoeComputeBackend
//                           src/ksana_llm/utils/config/model_config.h:36-212 (the members the factories read)
//   WeightStatus            src/ksana_llm/weight_status.h:16-19
//   BaseWeight              src/ksana_llm/models/base/base_weight.h:14-22 (GetModelWeights only)
//   Singleton               src/ksana_llm/utils/singleton.h
#pragma once

#ifdef KSQ_IN_KSANA_TREE
#  include "ksana_llm/models/common_moe/moe_config.h"
#  include "ksana_llm/models/base/base_weight.h"
#  include "ksana_llm/utils/context.h"
#  include "ksana_llm/utils/singleton.h"
#  include "ksana_llm/utils/status.h"
#  include "ksana_llm/utils/tensor.h"
#else

#  include <hip/hip_runtime_api.h>

#  include <any>
#  include <cstdint>
#  include <cstdio>
#  include <memory>
#  include <sstream>
#  include <stdexcept>
#  include <string>
#  include <unordered_map>
#  include <vector>

namespace ksana_llm {

enum RetCode { RET_SUCCESS = 0, RET_INVALID_ARGUMENT = 1, RET_RUNTIME_FAILED = 2, RET_UNDEFINED_REFERENCE = 3 };

class Status {
 public:
  Status() = default;
  explicit Status(RetCode code, const std::string& message = "") : code_(code), message_(message) {}
  bool OK() const { return code_ == RET_SUCCESS; }
  RetCode GetCode() const { return code_; }
  const std::string& GetMessage() const { return message_; }
  std::string ToString() const { return OK() ? "OK" : message_; }

 private:
  RetCode code_ = RET_SUCCESS;
  std::string message_;
};

#  define STATUS_CHECK_FAILURE(expr) \
    do {                             \
      Status _s = (expr);            \
      if (!_s.OK()) return _s;       \
    } while (0)

#  define KLLM_THROW(msg) throw std::runtime_error(std::string(msg))
#  define KLLM_CHECK_WITH_INFO(cond, msg) \
    do {                                  \
      if (!(cond)) KLLM_THROW(msg);       \
    } while (0)

enum DataType {
  TYPE_INVALID,
  TYPE_BOOL,
  TYPE_UINT8,
  TYPE_UINT16,
  TYPE_UINT32,
  TYPE_UINT64,
  TYPE_INT8,
  TYPE_INT16,
  TYPE_INT32,
  TYPE_INT64,
  TYPE_BF16,
  TYPE_FP16,
  TYPE_FP32,
  TYPE_FP64,
  TYPE_BYTES,
  TYPE_FP8_E4M3,
  TYPE_I4_GROUP,
  TYPE_BLOCK_FP8_E4M3,
  TYPE_FP8_E5M2,
  TYPE_VOID,
  TYPE_POINTER,
  TYPE_UINT4x2,
  TYPE_INT4x2,
  TYPE_FP8_DS_MLA
};

inline size_t GetTypeSize(DataType dtype) {
  switch (dtype) {
    case TYPE_BOOL:
    case TYPE_UINT8:
    case TYPE_INT8:
    case TYPE_BYTES:
    case TYPE_FP8_E4M3:
    case TYPE_FP8_E5M2:
    case TYPE_BLOCK_FP8_E4M3:
    case TYPE_I4_GROUP:
    case TYPE_UINT4x2:
    case TYPE_INT4x2:
    case TYPE_FP8_DS_MLA:
      return 1;
    case TYPE_UINT16:
    case TYPE_INT16:
    case TYPE_BF16:
    case TYPE_FP16:
      return 2;
    case TYPE_UINT32:
    case TYPE_INT32:
    case TYPE_FP32:
      return 4;
    case TYPE_UINT64:
    case TYPE_INT64:
    case TYPE_FP64:
    case TYPE_POINTER:
      return 8;
    default:
      return 0;
  }
}

enum class MemoryLocation { LOCATION_UNKNOWN, LOCATION_HOST, LOCATION_DEVICE };

// Device (or host) buffer with a shape.  Owns its memory when constructed without a pointer.
class Tensor {
 public:
  MemoryLocation location = MemoryLocation::LOCATION_UNKNOWN;
  DataType dtype = TYPE_INVALID;
  std::vector<size_t> shape;
  int device_id = 0;

  // quantization side tensors, named as in the reference
  std::shared_ptr<Tensor> scales, zeros, g_idx, perm, input_scales, weight_scales, pre_quant_scales, input_alpha;
  float alpha = 1.0f;  // W4A8: input_scale * weight_scale_2

  Tensor() = default;
  Tensor(MemoryLocation location, DataType dtype, const std::vector<size_t>& shape, int device_id,
         void* refer_ptr = nullptr)
      : location(location), dtype(dtype), shape(shape), device_id(device_id) {
    if (refer_ptr) {
      ptr_ = refer_ptr;
      return;
    }
    size_t bytes = GetTotalBytes();
    if (bytes == 0) return;
    void* p = nullptr;
    if (location == MemoryLocation::LOCATION_DEVICE) {
      if (hipMalloc(&p, bytes) != hipSuccess) KLLM_THROW("Tensor: hipMalloc failed");
      owner_ = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
    } else {
      if (hipHostMalloc(&p, bytes, hipHostMallocDefault) != hipSuccess) KLLM_THROW("Tensor: hipHostMalloc failed");
      owner_ = std::shared_ptr<void>(p, [](void* q) { (void)hipHostFree(q); });
    }
    ptr_ = p;
  }

  size_t GetElementNumber() const {
    if (shape.empty()) return 0;
    size_t n = 1;
    for (size_t d : shape) n *= d;
    return n;
  }
  size_t GetTotalBytes() const { return GetElementNumber() * GetTypeSize(dtype); }

  template <typename T>
  T* GetPtr() const {
    return reinterpret_cast<T*>(ptr_);
  }

 private:
  void* ptr_ = nullptr;
  std::shared_ptr<void> owner_;
};

class Stream {
 public:
  explicit Stream(hipStream_t s = nullptr) : stream_(s) {}
  hipStream_t& Get() { return stream_; }

 private:
  hipStream_t stream_;
};

struct BaseLayerParameters {};

enum QuantMode {
  QUANT_NONE,
  QUANT_GPTQ,
  QUANT_AWQ,
  QUANT_FP8_E4M3,
  QUANT_BLOCK_FP8_E4M3,
  QUANT_W4A8_AWQ,
  MOE_QUANT_NONE,
  MOE_QUANT_BLOCK_FP8_E4M3,
  MOE_QUANT_FP8_E4M3,
  MOE_QUANT_GPTQ
};
enum LinearComputeBackend {
  DEFAULT_LINEAR_BACKEND,
  CUTLASS_LINEAR_BACKEND,
  MARLIN_LINEAR_BACKEND,
  MACHETE_LINEAR_BACKEND
};
enum MoeComputeBackend { DEFAULT_MOE_BACKEND, CUTLASS_MOE_BACKEND, MARLIN_MOE_BACKEND, TRITON_MOE_BACKEND };
enum class W4AFP8_MOE_BACKEND { Default, GroupTriton, TensorTriton };

// What the loader records about one weight (src/ksana_llm/weight_status.h:16-19): W4A8 weights carry their n and k here.
struct WeightStatus {
  QuantMode quant_mode = QuantMode::QUANT_NONE;
  std::unordered_map<std::string, size_t> layout;
};

class Context {
 public:
  explicit Context(int tensor_parallel_size = 1, hipStream_t compute_stream = nullptr)
      : tp_(tensor_parallel_size), compute_streams_(static_cast<size_t>(tensor_parallel_size), Stream(compute_stream)) {}
  int GetTensorParallelSize() const { return tp_; }
  std::vector<Stream>& GetComputeStreams() { return compute_streams_; }
  void SetWeightStatus(const std::string& key, const WeightStatus& status) { weight_status_map_[key] = status; }
  WeightStatus& GetWeightStatus(const std::string& key) { return weight_status_map_[key]; }  // default entry if absent

 private:
  int tp_;
  std::vector<Stream> compute_streams_;
  std::unordered_map<std::string, WeightStatus> weight_status_map_;
};

// The part of the model-weight interface the factories use (src/ksana_llm/models/base/base_weight.h:14-22).
class BaseWeight {
 public:
  virtual ~BaseWeight() {}
  virtual Tensor GetModelWeights(const std::string& weight_name) = 0;
};
enum class MoeScaleNormMode { NO_NORM = 0, RE_NORM = 1 };

struct QuantConfig {
  QuantMode method = QUANT_NONE;
  size_t bits = 4;
  size_t group_size = 128;
  bool desc_act = false;
  std::vector<size_t> weight_block_size{128, 128};
  LinearComputeBackend backend = CUTLASS_LINEAR_BACKEND;
  bool is_fp8_blockwise = false;
  std::vector<std::string> pattern_layers;
  std::vector<std::string> ignored_layers;
};

struct MoeConfig {
  size_t num_experts = 1;
  size_t experts_topk = 1;
  size_t moe_inter_size = 0;
  size_t shared_expert_inter_size = 0;
  uint32_t num_expert_group = 1;
  uint32_t expert_groups_topk = 1;
  std::string scoring_func = "softmax";
  std::string topk_method = "greedy";
  bool norm_topk_prob = false;
  bool use_e_score_correction_bias = false;
  float routed_scaling_factor = 1.0f;
  bool use_vllm_moe = false;
  bool apply_weight = false;
};

struct MlaConfig {
  uint32_t q_lora_rank = 0;
  uint32_t kv_lora_rank = 0;
  uint32_t qk_nope_head_dim = 0;
  uint32_t qk_rope_head_dim = 0;
  uint32_t v_head_dim = 0;
};

struct ModelConfig {
  std::string type;
  bool is_quant = false;
  QuantConfig quant_config;
  std::vector<QuantConfig> sub_quant_configs;
  size_t hidden_units = 0;
  size_t inter_size = 0;
  size_t head_num = 0;
  size_t num_key_value_heads = 0;
  size_t size_per_head = 0;
  MoeConfig moe_config;
  MlaConfig mla_config;
};

struct ParallelismBasicConfig {
  size_t tensor_parallel_size = 1;
  size_t attn_data_parallel_size = 1;
  size_t attn_tensor_parallel_size = 1;
  size_t expert_parallel_size = 1;
  size_t expert_world_size = 1;
  size_t moe_tensor_para_size = 1;
};

struct RuntimeConfig {
  ParallelismBasicConfig parallel_basic_config;
  DataType inter_data_type = TYPE_FP16;
  size_t max_batch_size = 256;
  size_t max_step_token_num = 4096;
  bool enable_full_shared_expert = false;
  W4AFP8_MOE_BACKEND w4afp8_moe_backend = W4AFP8_MOE_BACKEND::Default;
};

template <typename T>
class Singleton {
 public:
  static std::shared_ptr<T> GetInstance() {
    static std::shared_ptr<T> instance = std::make_shared<T>();
    return instance;
  }
};

}  // namespace ksana_llm
#endif  // KSQ_IN_KSANA_TREE
