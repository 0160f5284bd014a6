#include "moe_layer.h"

#include <algorithm>

namespace ksana_llm {

static inline size_t AlignAddress(size_t size) { return (size + 255) & ~static_cast<size_t>(255); }

Status MoeLayer::Init(const std::vector<std::any>& parameters, const RuntimeConfig& runtime_config,
                      std::shared_ptr<Context> context, int rank) {
  STATUS_CHECK_FAILURE(BaseLayer::Init(parameters, runtime_config, context, rank));
  if (parameters.size() < 21) return Status(RET_INVALID_ARGUMENT, "MoeLayer: expects 21 init parameters");
  int parameter_index = 0;
  moe_scale_norm_mode_ = std::any_cast<const MoeScaleNormMode>(parameters[parameter_index++]);
  max_token_num_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  layer_idx_ = std::any_cast<const int>(parameters[parameter_index++]);
  expert_num_per_node_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  expert_hidden_size_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  expert_inter_size_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  expert_topk_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  tp_size_ = static_cast<int>(std::any_cast<const size_t>(parameters[parameter_index++]));
  use_vllm_moe_ = std::any_cast<const bool>(parameters[parameter_index++]);
  num_expert_group_ = std::any_cast<const uint32_t>(parameters[parameter_index++]);
  expert_groups_topk_ = std::any_cast<const uint32_t>(parameters[parameter_index++]);
  scoring_func_ = std::any_cast<const std::string>(parameters[parameter_index++]);
  topk_method_ = std::any_cast<const std::string>(parameters[parameter_index++]);
  norm_topk_prob_ = std::any_cast<const bool>(parameters[parameter_index++]);
  routed_scaling_factor_ = std::any_cast<const float>(parameters[parameter_index++]);
  use_e_score_correction_bias_ = std::any_cast<const bool>(parameters[parameter_index++]);
  [[maybe_unused]] bool enable_full_shared_expert = std::any_cast<const bool>(parameters[parameter_index++]);
  DataType fp8_weight_dtype = std::any_cast<DataType>(parameters[parameter_index++]);
  DataType int_weight_dtype = std::any_cast<DataType>(parameters[parameter_index++]);
  group_size_ = std::any_cast<int>(parameters[parameter_index++]);
  apply_weight_ = std::any_cast<bool>(parameters[parameter_index++]);

  // weight / compute type resolution of the reference (moe_layer.cpp:66-86): the block-fp8 and the int4 rows
  weight_dtype_ = inter_data_type_;
  compute_dtype_ = inter_data_type_;
  if (fp8_weight_dtype == TYPE_BLOCK_FP8_E4M3) {
    weight_dtype_ = TYPE_FP8_E4M3;
    compute_dtype_ = TYPE_BLOCK_FP8_E4M3;
    if (int_weight_dtype == TYPE_UINT4x2 || int_weight_dtype == TYPE_INT4x2)
      return Status(RET_INVALID_ARGUMENT, "MoeLayer: int4 weights with fp8 activations (w4afp8) are not built");
    if (expert_hidden_size_ % 128 != 0 || expert_inter_size_ % 128 != 0)
      return Status(RET_INVALID_ARGUMENT, "MoeLayer: block-fp8 experts need hidden and inter sizes that are multiples of 128");
  } else if (fp8_weight_dtype == TYPE_FP8_E4M3) {
    return Status(RET_INVALID_ARGUMENT, "MoeLayer: per-tensor fp8 expert weights are not built on this path");
  } else if (int_weight_dtype == TYPE_UINT4x2 || int_weight_dtype == TYPE_INT4x2) {
    weight_dtype_ = int_weight_dtype;
  } else {
    return Status(RET_INVALID_ARGUMENT, "MoeLayer: only int4 (TYPE_UINT4x2 / TYPE_INT4x2) or block-fp8 expert weights are built");
  }
  if (!use_vllm_moe_) return Status(RET_INVALID_ARGUMENT, "MoeLayer: only the use_vllm_moe flow is built");
  if (scoring_func_ != "softmax" && scoring_func_ != "sigmoid") {
    return Status(RET_INVALID_ARGUMENT, "MoeLayer: unsupported scoring function: " + scoring_func_);
  }
  if (num_expert_group_ == 0 || num_expert_group_ > 64 || expert_num_per_node_ % num_expert_group_ != 0 ||
      expert_groups_topk_ == 0 || expert_groups_topk_ > num_expert_group_ ||
      expert_topk_ > expert_groups_topk_ * (expert_num_per_node_ / num_expert_group_)) {
    return Status(RET_INVALID_ARGUMENT, "MoeLayer: expert groups must divide the experts (at most 64 groups) and the "
                                        "kept groups must hold at least topk experts");
  }
  if (runtime_config.parallel_basic_config.expert_parallel_size * runtime_config.parallel_basic_config.expert_world_size != 1) {
    return Status(RET_INVALID_ARGUMENT, "MoeLayer: expert parallelism is not built");
  }
  if (!IsFp8() && group_size_ != 128) return Status(RET_INVALID_ARGUMENT, "MoeLayer: expert group size must be 128");
  if (expert_topk_ == 0 || expert_topk_ > 32 || expert_num_per_node_ > 1024 || expert_topk_ > expert_num_per_node_) {
    return Status(RET_INVALID_ARGUMENT, "MoeLayer: need 1 <= topk <= min(32, experts), experts <= 1024");
  }
  return Status();
}

size_t MoeLayer::GetWorkspaceSize() {
  const size_t elem = GetTypeSize(inter_data_type_);
  const size_t m = std::min(kChunk, max_token_num_);
  const size_t numel = m * expert_topk_;
  size_t capacity = 0;
  for (size_t bm : {size_t(16), size_t(32), size_t(128), size_t(256)}) capacity = std::max(capacity, ksq_moe_align_capacity(numel, expert_num_per_node_, bm));
  topk_weights_size_ = AlignAddress(max_token_num_ * expert_topk_ * sizeof(float));
  topk_ids_size_ = AlignAddress(max_token_num_ * expert_topk_ * sizeof(int32_t));
  // sorted_ids [capacity] + expert_ids [capacity / 16] + num_tokens_post_pad [1]
  fused_id_buffer_size_ = AlignAddress((capacity + capacity / 16 + 1) * sizeof(int32_t));
  align_scratch_size_ = AlignAddress(ksq_moe_align_scratch_bytes(numel, expert_num_per_node_));
  cache1_size_ = AlignAddress(numel * expert_inter_size_ * 2 * elem);
  cache2_size_ = AlignAddress(numel * expert_inter_size_ * elem);
  if (IsFp8()) {
    // cache2 holds the quantized silu*mul output (codes, then scales); a1 the quantized hidden states of a chunk
    a2_q_size_ = AlignAddress(numel * expert_inter_size_);
    cache2_size_ = a2_q_size_ + AlignAddress(numel * (expert_inter_size_ / 128) * sizeof(float));
    a1_q_size_ = AlignAddress(m * expert_hidden_size_);
    a1_size_ = a1_q_size_ + AlignAddress(m * (expert_hidden_size_ / 128) * sizeof(float));
  }
  cache3_size_ = AlignAddress(numel * expert_hidden_size_ * elem);
  cache13_size_ = std::max(cache1_size_, cache3_size_);  // cache1 is dead once silu*mul has run: cache3 reuses it
  act_order1_size_ = reserve_act_order_ ? AlignAddress(numel * expert_hidden_size_ * elem) : 0;
  act_order2_size_ = reserve_act_order_ ? AlignAddress(numel * expert_inter_size_ * elem) : 0;
  max_ws_bytes_ = topk_weights_size_ + topk_ids_size_ + fused_id_buffer_size_ + align_scratch_size_ + cache13_size_ +
                  cache2_size_ + a1_size_ + act_order1_size_ + act_order2_size_;
  return max_ws_bytes_;
}

Status MoeLayer::SetWorkspaceBuffer(const std::shared_ptr<Tensor>& workspace_buffer) {
  workspace_buffer_ = workspace_buffer;
  return Status();
}

Status MoeLayer::Preprocess(const ModelConfig& model_config, const RuntimeConfig& runtime_config) {
  ksq_tile_desc desc;
  const int dtype = KsqDtype(inter_data_type_, "MoeLayer");
  if (IsFp8()) {
    if (ksq_select_tile(KSQ_KIND_FP8_BLOCKWISE, 1, expert_inter_size_ * 2, expert_hidden_size_, dtype, &desc) != KSQ_OK ||
        ksq_select_tile(KSQ_KIND_FP8_BLOCKWISE, 1, expert_hidden_size_, expert_inter_size_, dtype, &desc) != KSQ_OK) {
      return Status(RET_INVALID_ARGUMENT, std::string("MoeLayer: ") + ksq_last_error_string());
    }
    return Status();
  }
  if (ksq_select_tile(KSQ_KIND_MOE_W4A16, 1, expert_inter_size_ * 2, expert_hidden_size_, dtype, &desc) != KSQ_OK ||
      ksq_select_tile(KSQ_KIND_MOE_W4A16, 1, expert_hidden_size_, expert_inter_size_, dtype, &desc) != KSQ_OK) {
    return Status(RET_INVALID_ARGUMENT, std::string("MoeLayer: ") + ksq_last_error_string());
  }
  return Status();
}

Status MoeLayer::Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) {
  if (input_tensors.size() < 4) KLLM_THROW("MoeLayer: expects hidden_states, gating_output, up_gate weight, down weight");
  if (!workspace_buffer_ || max_ws_bytes_ == 0 || workspace_buffer_->GetTotalBytes() < max_ws_bytes_) {
    KLLM_THROW("MoeLayer: workspace buffer missing or smaller than GetWorkspaceSize()");
  }
  const size_t num_tokens = input_tensors[0].shape[0];
  const size_t hidden_size = input_tensors[0].shape[1];
  if (hidden_size != expert_hidden_size_) KLLM_THROW("MoeLayer: hidden size mismatch");
  if (num_tokens > max_token_num_) KLLM_THROW("MoeLayer: more tokens than max_token_num");
  if (IsFp8()) {
    if (!input_tensors[2].weight_scales || !input_tensors[3].weight_scales)
      KLLM_THROW("MoeLayer: block-fp8 expert weights have no weight_scales bound");
  } else if (!input_tensors[2].scales || !input_tensors[3].scales) {
    KLLM_THROW("MoeLayer: expert weights have no scales bound");
  }
  if ((input_tensors[2].perm || input_tensors[3].perm) && (IsFp8() || !reserve_act_order_)) {
    KLLM_THROW("MoeLayer: act-order experts (perm bound to the weights) need the Marlin MoE layer");
  }

  const int dtype = KsqDtype(inter_data_type_, "MoeLayer");
  const size_t elem = GetTypeSize(inter_data_type_);
  hipStream_t stream = context_->GetComputeStreams()[rank_].Get();

  char* p = workspace_buffer_->GetPtr<char>();
  float* topk_weights = reinterpret_cast<float*>(p);
  p += topk_weights_size_;
  int32_t* topk_ids = reinterpret_cast<int32_t*>(p);
  p += topk_ids_size_;
  int32_t* id_buffer = reinterpret_cast<int32_t*>(p);
  p += fused_id_buffer_size_;
  void* align_scratch = p;
  p += align_scratch_size_;
  char* cache1 = p;
  char* cache3 = p;
  p += cache13_size_;
  char* cache2 = p;
  p += cache2_size_;
  char* a1 = p;  // block-fp8 only
  p += a1_size_;
  char* act_order1 = p;  // act-order experts only
  p += act_order1_size_;
  char* act_order2 = p;

  const int gating_dtype = input_tensors[1].dtype == TYPE_FP32 ? KSQ_F32 : KsqDtype(input_tensors[1].dtype, "MoeLayer");
  // the routers take norm_topk_prob alone, as in the reference's grouped-top-k flow (moe_layer.cpp:105-109);
  // moe_scale_norm_mode belongs to the reference's Cutlass MoE flow, which is not the one built here
  const bool renormalize = norm_topk_prob_;
  // routing (MoeLayer::ExecuteGroupedTopk of the reference, moe_layer.cpp:380-420): the correction bias is input 5
  const void* e_bias = nullptr;
  if (use_e_score_correction_bias_) {
    if (input_tensors.size() <= 5) KLLM_THROW("MoeLayer: use_e_score_correction_bias needs the bias as input tensor 5");
    if (input_tensors[5].dtype != TYPE_FP32) KLLM_THROW("MoeLayer: e_score_correction_bias must be fp32");
    e_bias = input_tensors[5].GetPtr<void>();
  }
  if (scoring_func_ == "softmax" && num_expert_group_ == 1 && !e_bias) {
    KsqCheck(ksq_moe_topk_softmax(input_tensors[1].GetPtr<void>(), topk_weights, topk_ids, num_tokens,
                                  expert_num_per_node_, expert_topk_, renormalize ? 1 : 0, routed_scaling_factor_,
                                  gating_dtype, stream),
             "MoeLayer");
  } else {
    KsqCheck(ksq_moe_grouped_topk(input_tensors[1].GetPtr<void>(), e_bias, topk_weights, topk_ids, num_tokens,
                                  expert_num_per_node_, expert_topk_, num_expert_group_, expert_groups_topk_,
                                  scoring_func_ == "sigmoid" ? KSQ_SCORE_SIGMOID : KSQ_SCORE_SOFTMAX,
                                  renormalize ? 1 : 0, routed_scaling_factor_, gating_dtype, stream),
             "MoeLayer");
  }

  const char* hidden = input_tensors[0].GetPtr<char>();
  char* out = output_tensors[0].GetPtr<char>();
  const void* w1 = input_tensors[2].GetPtr<void>();
  const void* w2 = input_tensors[3].GetPtr<void>();
  const void* w1_scale = IsFp8() ? input_tensors[2].weight_scales->GetPtr<void>() : input_tensors[2].scales->GetPtr<void>();
  const void* w2_scale = IsFp8() ? input_tensors[3].weight_scales->GetPtr<void>() : input_tensors[3].scales->GetPtr<void>();
  const size_t E = expert_num_per_node_, topk = expert_topk_, inter = expert_inter_size_;

  for (size_t begin = 0; begin < num_tokens; begin += kChunk) {
    const size_t tokens = std::min(kChunk, num_tokens - begin);
    const size_t numel = tokens * topk;
    const size_t block_m = BlockM(tokens);
    const size_t capacity = ksq_moe_align_capacity(numel, E, block_m);
    int32_t* sorted_ids = id_buffer;
    int32_t* expert_ids = sorted_ids + capacity;
    int32_t* num_post_pad = expert_ids + capacity / block_m;
    const int32_t* ids = topk_ids + begin * topk;
    const float* weights = topk_weights + begin * topk;

    const bool few = tokens <= kFewTokens && numel <= 64 && !input_tensors[2].perm && !input_tensors[3].perm &&
                     (2 * inter) % 32 == 0 && topk <= 32;
    if (!few) KsqCheck(ksq_moe_align(ids, numel, E, block_m, sorted_ids, expert_ids, num_post_pad, align_scratch, stream), "MoeLayer");
    if (IsFp8()) {
      // InvokeFusedMoeKernelFunc with compute_dtype TYPE_BLOCK_FP8_E4M3 (moe_kernel_wrapper.cpp:435-456): activations
      // are quantized per token and 128 channels (scales [rows, k/128]) in front of each GEMM, silu*mul fused into
      // the second quantization
      void* a1_s = a1 + a1_q_size_;
      void* a2_s = cache2 + a2_q_size_;
      KsqCheck(ksq_fp8_group_quant(hidden + begin * hidden_size * elem, a1, a1_s, tokens, hidden_size, 128, 0, 0, dtype, stream),
               "MoeLayer");
      if (few) {  // a few decode tokens: no aligned permutation, the sum over top-k inside the second GEMM
        KsqCheck(ksq_moe_fp8_blockwise_gemm(cache1, a1, a1_s, 0, tokens, w1, w1_scale, nullptr, nullptr, ids, nullptr, numel,
                                            topk, E, 2 * inter, hidden_size, 16, dtype, stream),
                 "MoeLayer");
        KsqCheck(ksq_fp8_group_quant(cache1, cache2, a2_s, numel, inter, 128, 0, 1, dtype, stream), "MoeLayer");
        KsqCheck(ksq_moe_fp8_down_sum(out + begin * hidden_size * elem, cache2, a2_s, w2, w2_scale, weights, ids, tokens, topk, E,
                                      hidden_size, inter, dtype, stream),
                 "MoeLayer");
        continue;
      }
      KsqCheck(ksq_moe_fp8_blockwise_gemm(cache1, a1, a1_s, 0, tokens, w1, w1_scale, nullptr, sorted_ids, expert_ids,
                                          num_post_pad, numel, topk, E, 2 * inter, hidden_size, block_m, dtype, stream),
               "MoeLayer");
      KsqCheck(ksq_fp8_group_quant(cache1, cache2, a2_s, numel, inter, 128, 0, 1, dtype, stream), "MoeLayer");
      KsqCheck(ksq_moe_fp8_blockwise_gemm(cache3, cache2, a2_s, 0, numel, w2, w2_scale, weights, sorted_ids, expert_ids,
                                          num_post_pad, numel, 1, E, hidden_size, inter, block_m, dtype, stream),
               "MoeLayer");
      KsqCheck(ksq_moe_sum(cache3, out + begin * hidden_size * elem, tokens, topk, hidden_size, dtype, stream), "MoeLayer");
      continue;
    }
    // A few decode tokens: two launches.  Every slot is a block of its own (no aligned permutation) in the first GEMM,
    // which applies the activation in its epilogue; the second GEMM carries the sum over top-k.
    if (few) {
      KsqCheck(ksq_moe_w4a16_gate_up_silu(cache2, hidden + begin * hidden_size * elem, w1, w1_scale, nullptr, nullptr, ids,
                                          nullptr, numel, topk, E, 2 * inter, hidden_size, group_size_, 16, dtype, stream),
               "MoeLayer");
      KsqCheck(ksq_moe_w4a16_down_sum(out + begin * hidden_size * elem, cache2, w2, w2_scale, weights, ids, tokens, topk, E,
                                      hidden_size, inter, group_size_, dtype, stream),
               "MoeLayer");
      continue;
    }
    // gate_up: every (token, slot) row reads hidden[token]; with act-order experts the row of a slot is gathered
    // through its expert's permutation first (the weight rows lie in that order) and the GEMM reads it by slot
    const void* gemm1_in = hidden + begin * hidden_size * elem;
    size_t gemm1_topk = topk;
    if (input_tensors[2].perm) {
      KsqCheck(ksq_moe_permute_columns(gemm1_in, input_tensors[2].perm->GetPtr<void>(), ids, act_order1, numel, hidden_size,
                                       topk, E, dtype, stream),
               "MoeLayer");
      gemm1_in = act_order1;
      gemm1_topk = 1;
    }
    // the activation runs in the first GEMM's epilogue, except with 128-row blocks (a size ksq_moe_block_m no longer
    // picks but a caller may ask for), where the two launches measured faster (64 rows per expert: 1.75 against 1.87 ms)
    if (block_m != 128 && (2 * inter) % 32 == 0) {
      KsqCheck(ksq_moe_w4a16_gate_up_silu(cache2, gemm1_in, w1, w1_scale, nullptr, sorted_ids, expert_ids, num_post_pad,
                                          numel, gemm1_topk, E, 2 * inter, hidden_size, group_size_, block_m, dtype, stream),
               "MoeLayer");
    } else {
      KsqCheck(ksq_moe_w4a16_gemm(cache1, gemm1_in, w1, w1_scale, nullptr, nullptr, sorted_ids, expert_ids, num_post_pad,
                                  numel, gemm1_topk, E, 2 * inter, hidden_size, group_size_, block_m, dtype, stream),
               "MoeLayer");
      KsqCheck(ksq_moe_silu_mul(cache1, cache2, numel, inter, dtype, stream), "MoeLayer");
    }
    // down: row s reads cache2[s]; the routing weight is applied in the epilogue
    const void* gemm2_in = cache2;
    if (input_tensors[3].perm) {
      KsqCheck(ksq_moe_permute_columns(cache2, input_tensors[3].perm->GetPtr<void>(), ids, act_order2, numel, inter, 1, E,
                                       dtype, stream),
               "MoeLayer");
      gemm2_in = act_order2;
    }
    KsqCheck(ksq_moe_w4a16_gemm(cache3, gemm2_in, w2, w2_scale, nullptr, weights, sorted_ids, expert_ids, num_post_pad,
                                numel, 1, E, hidden_size, inter, group_size_, block_m, dtype, stream),
             "MoeLayer");
    KsqCheck(ksq_moe_sum(cache3, out + begin * hidden_size * elem, tokens, topk, hidden_size, dtype, stream), "MoeLayer");
  }
  output_tensors[0].shape = {num_tokens, hidden_size};
  output_tensors[0].dtype = input_tensors[0].dtype;
  return Status();
}

}  // namespace ksana_llm
