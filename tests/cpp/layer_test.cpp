// Driver for the C++ layer classes: builds every layer the way model code does - MatMulLayerFactory::AutoCreateLayer /
// MoeLayerFactory::AutoCreateMoeLayer from a weight name, the loaded weight and a model configuration - feeds it the raw
// tensors found in a directory and writes the output next to them.  tests/test_gpu_layers.py creates the inputs,
// runs this program and compares the output with the CPU oracle.
//
//   layer_test w4a16     <dir> <gptq|awq> <f16|bf16> <cutlass|marlin|machete> m n k group
//   layer_test blockwise <dir> <f16|bf16> m n k fuse_silu_mul
//   (w4a16: an optional trailing 1 = GPTQ act-order, g_idx.bin int32 [k])
//   layer_test fp8_tensor <dir> <f16|bf16> m n k static
//   layer_test moe       <dir> <f16|bf16> tokens experts hidden inter topk renorm scaling [groups topk_group scoring use_bias]
//   layer_test moe_fp8   <dir> <f16|bf16> tokens experts hidden inter topk renorm scaling
//   layer_test marlin_moe <dir> f16 tokens experts hidden inter topk renorm
//   layer_test errors
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <map>

#include "blockwise_matmul_layer.h"
#include "layer_factory.h"
#include "finegrained_mixed_dtype_gemm_layer.h"
#include "fp8_matmul_layer.h"
#include "moe_layer.h"
#include "marlin_moe_layer.h"
#include "quant_weight_repack.h"
#include "w4a16_matmul_layer.h"

using namespace ksana_llm;

#define HIP_OK(expr)                                                                      \
  do {                                                                                    \
    hipError_t _e = (expr);                                                               \
    if (_e != hipSuccess) {                                                               \
      std::fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(_e));              \
      std::exit(2);                                                                       \
    }                                                                                     \
  } while (0)

static std::vector<char> ReadFile(const std::string& path) {
  std::ifstream f(path, std::ios::binary | std::ios::ate);
  if (!f) {
    std::fprintf(stderr, "cannot open %s\n", path.c_str());
    std::exit(2);
  }
  std::vector<char> buf(static_cast<size_t>(f.tellg()));
  f.seekg(0);
  f.read(buf.data(), static_cast<std::streamsize>(buf.size()));
  return buf;
}

static Tensor Upload(const std::string& path, DataType dtype, const std::vector<size_t>& shape) {
  std::vector<char> host = ReadFile(path);
  Tensor t(MemoryLocation::LOCATION_DEVICE, dtype, shape, 0);
  if (host.size() != t.GetTotalBytes()) {
    std::fprintf(stderr, "%s: %zu bytes on disk, %zu expected\n", path.c_str(), host.size(), t.GetTotalBytes());
    std::exit(2);
  }
  HIP_OK(hipMemcpy(t.GetPtr<void>(), host.data(), host.size(), hipMemcpyHostToDevice));
  return t;
}

static void Download(const Tensor& t, const std::string& path) {
  std::vector<char> host(t.GetTotalBytes());
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(host.data(), t.GetPtr<void>(), host.size(), hipMemcpyDeviceToHost));
  std::ofstream f(path, std::ios::binary);
  f.write(host.data(), static_cast<std::streamsize>(host.size()));
}

// the model weights the factories look up by name
class TestWeights : public BaseWeight {
 public:
  Tensor GetModelWeights(const std::string& weight_name) override {
    auto it = weights.find(weight_name);
    return it == weights.end() ? Tensor() : it->second;
  }
  std::map<std::string, Tensor> weights;
};

static DataType ParseT(const char* s) {
  return std::strcmp(s, "bf16") == 0 ? TYPE_BF16 : (std::strcmp(s, "f32") == 0 ? TYPE_FP32 : TYPE_FP16);
}

static void Drive(std::shared_ptr<BaseLayer> layer, const ModelConfig& mc, const RuntimeConfig& rc,
                  const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  size_t ws = layer->GetWorkspaceSize();
  auto buffer = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_INT8, std::vector<size_t>{ws ? ws : 256}, 0);
  Status s = layer->SetWorkspaceBuffer(buffer);
  if (!s.OK()) KLLM_THROW(s.GetMessage());
  s = layer->Preprocess(mc, rc);
  if (!s.OK()) KLLM_THROW(s.GetMessage());
  s = layer->Forward(inputs, outputs);
  if (!s.OK()) KLLM_THROW(s.GetMessage());
}

static int RunW4A16(int argc, char** argv) {
  if (argc < 10) return 2;
  const std::string dir = argv[2];
  const bool awq = std::strcmp(argv[3], "awq") == 0;
  const DataType T = ParseT(argv[4]);
  const std::string be = argv[5];
  const size_t m = std::atol(argv[6]), n = std::atol(argv[7]), k = std::atol(argv[8]), group = std::atol(argv[9]);
  LinearComputeBackend backend = be == "marlin" ? MARLIN_LINEAR_BACKEND : be == "machete" ? MACHETE_LINEAR_BACKEND : CUTLASS_LINEAR_BACKEND;
  const bool desc_act = argc > 10 && std::atoi(argv[10]) != 0;  // GPTQ act-order: g_idx.bin int32 [k]

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  auto context = std::make_shared<Context>(1, stream);
  ModelConfig mc;
  mc.is_quant = true;
  mc.quant_config.method = awq ? QUANT_AWQ : QUANT_GPTQ;
  mc.quant_config.group_size = group;
  mc.quant_config.desc_act = desc_act;
  RuntimeConfig rc;
  rc.inter_data_type = T;
  rc.max_step_token_num = m;

  Tensor qweight = awq ? Upload(dir + "/qweight.bin", TYPE_INT32, {k, n / 8}) : Upload(dir + "/qweight.bin", TYPE_INT32, {k / 8, n});
  // argv[11] = 1: the tensors are one rank's K range of an act-order checkpoint twice as deep (scales.bin then holds the
  // scales of all 2k/group groups, g_idx.bin the checkpoint-wide group numbers of the range's rows)
  const bool k_range = argc > 11 && std::atoi(argv[11]) != 0;
  Tensor scales = Upload(dir + "/scales.bin", T, {(k_range ? 2 * k : k) / group, n});
  Tensor qzeros;
  if (awq) qzeros = Upload(dir + "/qzeros.bin", TYPE_INT32, {k / group, n / 8});
  Tensor g_idx;
  if (desc_act) g_idx = Upload(dir + "/g_idx.bin", TYPE_INT32, {k});
  Tensor weight = PackGroupQuantWeight(qweight, scales, awq ? &qzeros : nullptr, mc.quant_config.method, group, 0, stream,
                                       desc_act ? &g_idx : nullptr, !k_range);

  // a column-parallel projection of a model with hidden size k and inter size n (mlp.gate_proj: all of K on this
  // rank), or - k_slice - the row-parallel mlp.down_proj of a model with inter size k and hidden size n, whose K is a
  // rank's slice of the checkpoint's
  const bool k_slice = k_range;
  // two tensor-parallel ranks, this is rank 0.  argv[12]: the size the context reports, where it differs from the cut the
  // factory applies (which follows the runtime configuration): the layer's workspace bound must not rest on the former
  const int context_tp = argc > 12 ? std::atoi(argv[12]) : 2;
  if (k_slice) context = std::make_shared<Context>(context_tp, stream);
  mc.hidden_units = k_slice ? n : k;
  mc.inter_size = k_slice ? 2 * k : n;
  const std::string name = k_slice ? "model.layers.0.mlp.down_proj.weight" : "model.layers.0.mlp.gate_proj.weight";
  auto weights = std::make_shared<TestWeights>();
  weights->weights[name] = weight;
  MatMulLayerFactory factory(mc, rc, 0, context);
  if (k_slice) rc.parallel_basic_config.tensor_parallel_size = 2;
  MatMulLayerFactory tp_factory(mc, rc, 0, context);
  auto layer = (k_slice ? tp_factory : factory).AutoCreateLayer(weights, name, TYPE_I4_GROUP, T, T, backend, {});
  Tensor x = Upload(dir + "/x.bin", T, {m, k});
  std::vector<Tensor> outputs{Tensor(MemoryLocation::LOCATION_DEVICE, T, {m, n}, 0)};
  Drive(layer, mc, rc, {x, weight}, outputs);
  if (outputs[0].shape != std::vector<size_t>{m, n} || outputs[0].dtype != T) return 3;
  HIP_OK(hipStreamSynchronize(stream));
  Download(outputs[0], dir + "/y.bin");
  return 0;
}

static int RunBlockwise(int argc, char** argv) {
  if (argc < 8) return 2;
  const std::string dir = argv[2];
  const DataType T = ParseT(argv[3]);
  const size_t m = std::atol(argv[4]), n = std::atol(argv[5]), k = std::atol(argv[6]);
  const bool fuse = std::atoi(argv[7]) != 0;
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  auto context = std::make_shared<Context>(1, stream);
  ModelConfig mc;
  mc.is_quant = true;
  mc.quant_config.method = QUANT_BLOCK_FP8_E4M3;
  RuntimeConfig rc;
  rc.inter_data_type = T;
  rc.max_step_token_num = argc > 8 ? std::atol(argv[8]) : (m + 3) / 4 * 4;  // optional: the layer's max_m

  Tensor loaded = Upload(dir + "/w.bin", TYPE_FP8_E4M3, {n, k});
  loaded.weight_scales = std::make_shared<Tensor>(Upload(dir + "/w_scale.bin", TYPE_FP32, {(n + 127) / 128, k / 128}));
  Tensor weight = PackFp8Weight(loaded, 0, stream);
  const std::string name = "model.layers.0.mlp.up_proj.weight";
  auto weights = std::make_shared<TestWeights>();
  weights->weights[name] = weight;
  mc.quant_config.weight_block_size = {128, 128};
  MatMulLayerFactory factory(mc, rc, 0, context);
  auto layer = factory.AutoCreateLayer(weights, name, TYPE_FP8_E4M3, T, T, DEFAULT_LINEAR_BACKEND, {false});  // skip_quant
  Tensor x = Upload(dir + "/x.bin", T, {m, fuse ? 2 * k : k});
  std::vector<Tensor> outputs{Tensor(MemoryLocation::LOCATION_DEVICE, T, {m, n}, 0)};
  Drive(layer, mc, rc, {x, weight}, outputs);
  HIP_OK(hipStreamSynchronize(stream));
  Download(outputs[0], dir + "/y.bin");
  return 0;
}

// per-tensor fp8: w.bin [n, k] e4m3, w_scale.bin 1 fp32, optional in_scale.bin 1 fp32 (static activation scale)
static int RunFp8Tensor(int argc, char** argv) {
  if (argc < 8) return 2;
  const std::string dir = argv[2];
  const DataType T = ParseT(argv[3]);
  const size_t m = std::atol(argv[4]), n = std::atol(argv[5]), k = std::atol(argv[6]);
  const bool is_static = std::atoi(argv[7]) != 0;
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  auto context = std::make_shared<Context>(1, stream);
  ModelConfig mc;
  RuntimeConfig rc;
  rc.inter_data_type = T;
  rc.max_step_token_num = m;
  Tensor loaded = Upload(dir + "/w.bin", TYPE_FP8_E4M3, {n, k});
  loaded.weight_scales = std::make_shared<Tensor>(Upload(dir + "/w_scale.bin", TYPE_FP32, {1}));
  if (is_static) loaded.input_scales = std::make_shared<Tensor>(Upload(dir + "/in_scale.bin", TYPE_FP32, {1}));
  Tensor weight = PackFp8Weight(loaded, 0, stream);
  const std::string name = "model.layers.0.mlp.up_proj.weight";
  auto weights = std::make_shared<TestWeights>();
  weights->weights[name] = weight;
  mc.is_quant = true;
  mc.quant_config.method = QUANT_FP8_E4M3;
  MatMulLayerFactory factory(mc, rc, 0, context);
  auto layer = factory.AutoCreateLayer(weights, name, TYPE_FP8_E4M3, T, T, DEFAULT_LINEAR_BACKEND, {});
  Tensor x = Upload(dir + "/x.bin", T, {m, k});
  std::vector<Tensor> outputs{Tensor(MemoryLocation::LOCATION_DEVICE, T, {m, n}, 0)};
  Drive(layer, mc, rc, {x, weight}, outputs);
  HIP_OK(hipStreamSynchronize(stream));
  Download(outputs[0], dir + "/y.bin");
  return 0;
}

// w4a8 <dir> <f16|bf16> <m> <n> <k> <per_channel> <alpha> [group]
// (group 64 is built from the parameter struct: the factory's weight-name path, like the reference's, knows 128 only)
static int RunW4A8(int argc, char** argv) {
  if (argc < 9) return 2;
  const std::string dir = argv[2];
  const DataType T = ParseT(argv[3]);
  const size_t m = std::atol(argv[4]), n = std::atol(argv[5]), k = std::atol(argv[6]);
  const bool per_channel = std::atoi(argv[7]) != 0;
  const float alpha = static_cast<float>(std::atof(argv[8]));
  const size_t group = argc > 9 ? std::atol(argv[9]) : 128;
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  auto context = std::make_shared<Context>(1, stream);
  ModelConfig mc;
  RuntimeConfig rc;
  rc.inter_data_type = T;
  rc.max_step_token_num = m;
  Tensor loaded = Upload(dir + "/w.bin", TYPE_INT8, {k, n / 2});
  loaded.weight_scales = std::make_shared<Tensor>(Upload(dir + "/w_scale.bin", TYPE_FP16, {k / group, n}));
  loaded.input_scales = std::make_shared<Tensor>(Upload(dir + "/in_scale.bin", TYPE_FP32, {1}));
  if (per_channel) loaded.pre_quant_scales = std::make_shared<Tensor>(Upload(dir + "/pqs.bin", TYPE_FP32, {k}));
  loaded.alpha = alpha;
  Tensor weight = PackW4A8Weight(loaded, 0, stream);
  // the loader's record of a W4A8 weight: the mode, and the logical n and k the packed tensor no longer shows
  const std::string name = "model.layers.0.mlp.up_proj.weight";
  WeightStatus status;
  status.quant_mode = QUANT_W4A8_AWQ;
  status.layout = {{"n", n}, {"k", k}};
  context->SetWeightStatus(name, status);
  auto weights = std::make_shared<TestWeights>();
  weights->weights[name] = weight;
  MatMulLayerFactory factory(mc, rc, 0, context);
  std::shared_ptr<BaseLayer> layer;
  if (group == 128) {
    layer = factory.AutoCreateLayer(weights, name, TYPE_I4_GROUP, T, T, CUTLASS_LINEAR_BACKEND, {});
  } else {
    FinegrainedMixedDtypeGemmLayerParameters param;
    param.m = m;
    param.n = n;
    param.k = k;
    param.group_size = group;
    param.has_zero = false;
    param.activation_type = TYPE_FP8_E4M3;
    param.output_type = T;
    layer = factory.CreateLayer(TYPE_I4_GROUP, T, T, {param}, QUANT_W4A8_AWQ, CUTLASS_LINEAR_BACKEND);
  }
  Tensor x = Upload(dir + "/x.bin", T, {m, k});
  std::vector<Tensor> outputs{Tensor(MemoryLocation::LOCATION_DEVICE, T, {m, n}, 0)};
  Drive(layer, mc, rc, {x, weight}, outputs);
  HIP_OK(hipStreamSynchronize(stream));
  Download(outputs[0], dir + "/y.bin");
  return 0;
}

// Model and runtime configuration of a MoE model with E experts.  renorm: 0 = NO_NORM and norm_topk_prob false,
// 1 = RE_NORM and norm_topk_prob true, 2 = RE_NORM with norm_topk_prob false (the routers follow norm_topk_prob alone).
static MoeScaleNormMode MoeModel(ModelConfig& mc, RuntimeConfig& rc, size_t tokens, size_t E, size_t hidden, size_t inter,
                                 size_t topk, int renorm_arg, float scaling, uint32_t groups = 1, uint32_t topk_group = 1,
                                 const std::string& scoring = "softmax", bool use_bias = false) {
  rc.max_step_token_num = tokens;
  mc.hidden_units = hidden;
  mc.moe_config.num_experts = E;
  mc.moe_config.experts_topk = topk;
  mc.moe_config.moe_inter_size = inter;
  mc.moe_config.use_vllm_moe = true;
  mc.moe_config.num_expert_group = groups;
  mc.moe_config.expert_groups_topk = topk_group;
  mc.moe_config.scoring_func = scoring;
  mc.moe_config.norm_topk_prob = renorm_arg == 1;
  mc.moe_config.routed_scaling_factor = scaling;
  mc.moe_config.use_e_score_correction_bias = use_bias;
  return renorm_arg != 0 ? MoeScaleNormMode::RE_NORM : MoeScaleNormMode::NO_NORM;
}

static std::shared_ptr<BaseLayer> AutoMoe(const ModelConfig& mc, const RuntimeConfig& rc, std::shared_ptr<Context> context,
                                          const Tensor& w13, const Tensor& w2, DataType T, MoeScaleNormMode mode) {
  auto weights = std::make_shared<TestWeights>();
  weights->weights["model.layers.3.mlp.experts.up_gate_proj.weight"] = w13;
  weights->weights["model.layers.3.mlp.experts.down_proj.weight"] = w2;
  MoeLayerFactory factory(mc, rc, 0, context);
  return factory.AutoCreateMoeLayer(weights, {"model.layers.3.mlp.experts.up_gate_proj.weight",
                                              "model.layers.3.mlp.experts.down_proj.weight"},
                                    w13.dtype, T, T, 3, {mode});
}

static int RunMoe(int argc, char** argv) {
  if (argc < 11) return 2;
  const std::string dir = argv[2];
  const DataType T = ParseT(argv[3]);
  const size_t tokens = std::atol(argv[4]), E = std::atol(argv[5]), hidden = std::atol(argv[6]), inter = std::atol(argv[7]),
               topk = std::atol(argv[8]);
  const int renorm = std::atoi(argv[9]);
  const float scaling = static_cast<float>(std::atof(argv[10]));
  // optional grouped routing: groups topk_group scoring use_bias (bias.bin: fp32 [E])
  const uint32_t groups = argc > 11 ? std::atoi(argv[11]) : 1, topk_group = argc > 12 ? std::atoi(argv[12]) : 1;
  const std::string scoring = argc > 13 ? argv[13] : "softmax";
  const bool use_bias = argc > 14 && std::atoi(argv[14]) != 0;
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  auto context = std::make_shared<Context>(1, stream);
  ModelConfig mc;
  RuntimeConfig rc;
  rc.inter_data_type = T;

  Tensor w13 = PackMoeExpertWeight(Upload(dir + "/w13.bin", TYPE_UINT8, {E, 2 * inter, hidden / 2}),
                                   Upload(dir + "/s13.bin", T, {E, 2 * inter, hidden / 128}), 128, 0, stream);
  Tensor w2 = PackMoeExpertWeight(Upload(dir + "/w2.bin", TYPE_UINT8, {E, hidden, inter / 2}),
                                  Upload(dir + "/s2.bin", T, {E, hidden, inter / 128}), 128, 0, stream);
  HIP_OK(hipStreamSynchronize(stream));
  mc.is_quant = true;
  mc.quant_config.method = QUANT_GPTQ;
  mc.quant_config.bits = 4;
  mc.quant_config.group_size = 128;
  const MoeScaleNormMode mode = MoeModel(mc, rc, tokens, E, hidden, inter, topk, renorm, scaling, groups, topk_group, scoring, use_bias);
  auto layer = AutoMoe(mc, rc, context, w13, w2, T, mode);
  Tensor x = Upload(dir + "/x.bin", T, {tokens, hidden});
  Tensor gating = Upload(dir + "/gating.bin", TYPE_FP32, {tokens, E});
  std::vector<Tensor> outputs{Tensor(MemoryLocation::LOCATION_DEVICE, T, {tokens, hidden}, 0)};
  std::vector<Tensor> inputs{x, gating, w13, w2};
  if (use_bias) {
    inputs.push_back(Tensor());  // input 4 (expert map) is not used on this path
    inputs.push_back(Upload(dir + "/bias.bin", TYPE_FP32, {E}));
  }
  Drive(layer, mc, rc, inputs, outputs);
  HIP_OK(hipStreamSynchronize(stream));
  Download(outputs[0], dir + "/y.bin");
  return 0;
}

// GPTQ experts behind the Marlin MoE interface (fp16): qw13.bin int32 [E, hidden/8, 2*inter], s13.bin [E, hidden/128,
// 2*inter], qw2.bin int32 [E, inter/8, hidden], s2.bin [E, inter/128, hidden], gating.bin fp16 [tokens, E]
static int RunMarlinMoe(int argc, char** argv) {
  if (argc < 10) return 2;
  const std::string dir = argv[2];
  const DataType T = ParseT(argv[3]);
  const size_t tokens = std::atol(argv[4]), E = std::atol(argv[5]), hidden = std::atol(argv[6]), inter = std::atol(argv[7]),
               topk = std::atol(argv[8]);
  const bool renorm = std::atoi(argv[9]) != 0;
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  auto context = std::make_shared<Context>(1, stream);
  ModelConfig mc;
  RuntimeConfig rc;
  rc.inter_data_type = T;
  // optional: act-order experts, g13.bin int32 [E, hidden] and g2.bin int32 [E, inter] (the checkpoints' g_idx)
  const bool act_order = argc > 10 && std::atoi(argv[10]) != 0;
  Tensor g13, g2;
  if (act_order) {
    g13 = Upload(dir + "/g13.bin", TYPE_INT32, {E, hidden});
    g2 = Upload(dir + "/g2.bin", TYPE_INT32, {E, inter});
  }
  Tensor w13 = PackGptqExpertWeight(Upload(dir + "/qw13.bin", TYPE_INT32, {E, hidden / 8, 2 * inter}),
                                    Upload(dir + "/s13.bin", T, {E, hidden / 128, 2 * inter}), 128, 0, stream,
                                    act_order ? &g13 : nullptr);
  Tensor w2 = PackGptqExpertWeight(Upload(dir + "/qw2.bin", TYPE_INT32, {E, inter / 8, hidden}),
                                   Upload(dir + "/s2.bin", T, {E, inter / 128, hidden}), 128, 0, stream,
                                   act_order ? &g2 : nullptr);
  HIP_OK(hipStreamSynchronize(stream));
  // GPTQ experts of a model that does not take the aligned-block flow (use_vllm_moe false): the Marlin MoE layer
  mc.is_quant = true;
  mc.quant_config.method = QUANT_GPTQ;
  mc.quant_config.bits = 4;
  mc.quant_config.group_size = 128;
  const MoeScaleNormMode mode = MoeModel(mc, rc, tokens, E, hidden, inter, topk, renorm ? 1 : 0, 1.0f);
  mc.moe_config.use_vllm_moe = false;
  mc.moe_config.norm_topk_prob = false;  // this layer's router follows the scale-norm mode
  auto layer = AutoMoe(mc, rc, context, w13, w2, T, mode);
  Tensor x = Upload(dir + "/x.bin", T, {tokens, hidden});
  Tensor gating = Upload(dir + "/gating.bin", T, {tokens, E});
  std::vector<Tensor> outputs{Tensor(MemoryLocation::LOCATION_DEVICE, T, {tokens, hidden}, 0)};
  Drive(layer, mc, rc, {x, gating, w13, w2}, outputs);
  HIP_OK(hipStreamSynchronize(stream));
  Download(outputs[0], dir + "/y.bin");
  // a group index without the permutation that goes with it is refused with a message, not run wrongly
  Tensor w13_bad = w13;
  w13_bad.perm = nullptr;
  w13_bad.g_idx = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_INT32, std::vector<size_t>{E, hidden}, 0);
  bool threw = false;
  try {
    std::vector<Tensor> in2{x, gating, w13_bad, w2};
    layer->Forward(in2, outputs);
  } catch (const std::exception&) {
    threw = true;
  }
  if (!threw) {
    std::fprintf(stderr, "FAILED: g_idx without perm was accepted\n");
    return 1;
  }
  return 0;
}

// block-fp8 experts: w13.bin [E, 2*inter, hidden] e4m3, s13.bin fp32 [E, 2*inter/128, hidden/128], w2.bin, s2.bin alike
static int RunMoeFp8(int argc, char** argv) {
  if (argc < 11) return 2;
  const std::string dir = argv[2];
  const DataType T = ParseT(argv[3]);
  const size_t tokens = std::atol(argv[4]), E = std::atol(argv[5]), hidden = std::atol(argv[6]), inter = std::atol(argv[7]),
               topk = std::atol(argv[8]);
  const bool renorm = std::atoi(argv[9]) != 0;
  const float scaling = static_cast<float>(std::atof(argv[10]));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  auto context = std::make_shared<Context>(1, stream);
  ModelConfig mc;
  RuntimeConfig rc;
  rc.inter_data_type = T;
  Tensor w13_loaded = Upload(dir + "/w13.bin", TYPE_FP8_E4M3, {E, 2 * inter, hidden});
  w13_loaded.weight_scales = std::make_shared<Tensor>(Upload(dir + "/s13.bin", TYPE_FP32, {E, (2 * inter + 127) / 128, hidden / 128}));
  Tensor w2_loaded = Upload(dir + "/w2.bin", TYPE_FP8_E4M3, {E, hidden, inter});
  w2_loaded.weight_scales = std::make_shared<Tensor>(Upload(dir + "/s2.bin", TYPE_FP32, {E, (hidden + 127) / 128, inter / 128}));
  Tensor w13 = PackFp8Weight(w13_loaded, 0, stream);
  Tensor w2 = PackFp8Weight(w2_loaded, 0, stream);
  mc.is_quant = true;
  mc.quant_config.method = QUANT_BLOCK_FP8_E4M3;
  mc.quant_config.is_fp8_blockwise = true;
  const MoeScaleNormMode mode = MoeModel(mc, rc, tokens, E, hidden, inter, topk, renorm ? 1 : 0, scaling);
  auto layer = AutoMoe(mc, rc, context, w13, w2, T, mode);
  Tensor x = Upload(dir + "/x.bin", T, {tokens, hidden});
  Tensor gating = Upload(dir + "/gating.bin", TYPE_FP32, {tokens, E});
  std::vector<Tensor> outputs{Tensor(MemoryLocation::LOCATION_DEVICE, T, {tokens, hidden}, 0)};
  Drive(layer, mc, rc, {x, gating, w13, w2}, outputs);
  HIP_OK(hipStreamSynchronize(stream));
  Download(outputs[0], dir + "/y.bin");
  return 0;
}

// error behaviour that needs no kernel launch
static int RunErrors() {
  auto context = std::make_shared<Context>(1, nullptr);
  ModelConfig mc;
  RuntimeConfig rc;
  int failures = 0;
  auto expect = [&](bool ok, const char* what) {
    if (!ok) {
      std::fprintf(stderr, "FAILED: %s\n", what);
      ++failures;
    }
  };
  auto throws = [](auto&& fn) {
    try {
      fn();
    } catch (const std::exception&) {
      return true;
    }
    return false;
  };
  MatMulLayerFactory factory(mc, rc, 0, context);
  // unknown combination
  expect(throws([&] { factory.CreateLayer(TYPE_I4_GROUP, TYPE_FP32, TYPE_FP32, {}, QUANT_GPTQ, CUTLASS_LINEAR_BACKEND); }),
         "fp32 activations have no int4 layer");
  // too few parameters
  {
    CutlassMatMulLayer layer;
    expect(!layer.Init({size_t(1)}, rc, context, 0).OK(), "short parameter list is rejected");
  }
  // act-order: accepted with the whole K range, rejected for a K slice and for AWQ; its workspace holds the
  // permuted activations
  {
    MarlinMatMulLayer layer, sliced, awq, plain;
    std::vector<std::any> p{size_t(16), size_t(256), size_t(256), size_t(128), false, true, true, true, TYPE_I4_GROUP};
    expect(layer.Init(p, rc, context, 0).OK(), "desc_act init");
    p[5] = false;
    expect(plain.Init(p, rc, context, 0).OK(), "plain gptq init");
    expect(layer.GetWorkspaceSize() >= plain.GetWorkspaceSize() + 16 * 256 * 2, "desc_act workspace holds permuted x");
    p[5] = true;
    p[6] = false;
    expect(sliced.Init(p, rc, context, 0).OK(), "desc_act with a K slice init");
    // every group of the checkpoint may have rows in the slice, each run padded to 32 rows: 256 + 31 * 2 rows -> 384
    expect(sliced.GetWorkspaceSize() >= plain.GetWorkspaceSize() + 16 * 384 * 2, "K-slice workspace holds the padded x");
    p[6] = true;
    p[4] = true;
    expect(!awq.Init(p, rc, context, 0).OK(), "desc_act with AWQ is rejected");
  }
  // wrong weight data type surfaces in GetWorkspaceSize, as in the reference
  {
    CutlassMatMulLayer layer;
    std::vector<std::any> p{size_t(16), size_t(256), size_t(256), size_t(128), false, false, true, true, TYPE_FP16};
    expect(layer.Init(p, rc, context, 0).OK(), "init with foreign weight type succeeds");
    expect(throws([&] { layer.GetWorkspaceSize(); }), "GetWorkspaceSize throws for a non-int4 weight type");
  }
  // shape with no kernel: k not a multiple of 128
  {
    MacheteMatMulLayer layer;
    std::vector<std::any> p{size_t(16), size_t(256), size_t(200), size_t(128), false, false, true, true, TYPE_I4_GROUP};
    expect(layer.Init(p, rc, context, 0).OK(), "init");
    expect(!layer.Preprocess(mc, rc).OK(), "Preprocess reports a shape without a kernel");
  }
  // blockwise: block size other than 128; forward without workspace
  {
    BlockwiseMatMulLayer layer;
    std::vector<std::any> p{size_t(16), size_t(256), size_t(256), size_t(64), Tensor()};
    expect(!layer.Init(p, rc, context, 0).OK(), "block size 64 is rejected");
    BlockwiseMatMulLayer layer2;
    std::vector<std::any> p2{size_t(16), size_t(256), size_t(256), size_t(128), Tensor()};
    expect(layer2.Init(p2, rc, context, 0).OK(), "blockwise init");
    expect(layer2.GetWorkspaceSize() >= 16 * 256 + 16 * 2 * 4, "blockwise workspace holds a_q and a_s");
    std::vector<Tensor> out{Tensor()};
    Tensor x(MemoryLocation::LOCATION_DEVICE, TYPE_FP16, {16, 256}, 0, reinterpret_cast<void*>(0x1000));
    expect(throws([&] { layer2.Forward({x, Tensor()}, out); }), "Forward without a workspace buffer throws");
  }
  // per-tensor fp8
  {
    Fp8MatMulLayer layer, bad;
    std::vector<std::any> p{size_t(64), size_t(512)};
    expect(layer.Init(p, rc, context, 0).OK(), "fp8 per-tensor init");
    expect(layer.GetWorkspaceSize() >= Fp8MatMulLayer::kGemmWorkspaceBytes + 64 * 512 + 4, "fp8 per-tensor workspace");
    std::vector<std::any> q{size_t(64), size_t(200)};
    expect(!bad.Init(q, rc, context, 0).OK(), "k = 200 is rejected");
    std::vector<Tensor> out{Tensor()};
    Tensor x(MemoryLocation::LOCATION_DEVICE, TYPE_FP16, {16, 512}, 0, reinterpret_cast<void*>(0x1000));
    Tensor w(MemoryLocation::LOCATION_DEVICE, TYPE_FP8_E4M3, {64, 512}, 0, reinterpret_cast<void*>(0x1000));
    expect(throws([&] { layer.Forward({x, w}, out); }), "Forward without a workspace buffer throws");
  }
  // w4a8: group size, zero points, activation type, shapes; forward without a workspace
  {
    FinegrainedMixedDtypeGemmLayerParameters good;
    good.m = 64;
    good.n = 256;
    good.k = 512;
    good.group_size = 128;
    good.activation_type = TYPE_FP8_E4M3;
    good.output_type = TYPE_BF16;
    FinegrainedMixedDtypeGemmLayer ok;
    expect(ok.Init({good}, rc, context, 0).OK(), "w4a8 init");
    expect(ok.GetWorkspaceSize() >= 64 * 512 + 64 * 4 * 4, "w4a8 workspace holds the quantized activations and their group sums");
    expect(ok.Preprocess(mc, rc).OK(), "w4a8 preprocess");
    auto bad = [&](auto edit, const char* what) {
      FinegrainedMixedDtypeGemmLayerParameters p = good;
      edit(p);
      FinegrainedMixedDtypeGemmLayer l;
      expect(!l.Init({p}, rc, context, 0).OK(), what);
    };
    bad([](auto& p) { p.group_size = 32; }, "w4a8 rejects group size 32");
    {
      FinegrainedMixedDtypeGemmLayerParameters p64 = good;
      p64.group_size = 64;
      FinegrainedMixedDtypeGemmLayer l64;
      expect(l64.Init({p64}, rc, context, 0).OK(), "w4a8 init with group size 64");
      expect(l64.GetWorkspaceSize() >= 64 * 512 + 64 * 8 * 4, "w4a8 workspace with group size 64 holds twice the group sums");
    }
    bad([](auto& p) { p.has_zero = true; }, "w4a8 rejects zero points");
    bad([](auto& p) { p.activation_type = TYPE_FP16; }, "w4a8 rejects a 16-bit activation type");
    bad([](auto& p) { p.k = 200; }, "w4a8 rejects k = 200");
    bad([](auto& p) { p.output_type = TYPE_FP32; }, "w4a8 rejects fp32 output");
    std::vector<Tensor> out{Tensor()};
    Tensor x(MemoryLocation::LOCATION_DEVICE, TYPE_BF16, {16, 512}, 0, reinterpret_cast<void*>(0x1000));
    Tensor w(MemoryLocation::LOCATION_DEVICE, TYPE_INT8, {512, 128}, 0, reinterpret_cast<void*>(0x1000));
    expect(throws([&] { ok.Forward({x, w}, out); }), "w4a8 Forward without a workspace buffer throws");
  }
  // marlin moe: fp16 only, 20 parameters
  {
    std::vector<std::any> p{MoeScaleNormMode::RE_NORM, size_t(8), size_t(8), size_t(256), size_t(128), size_t(2), size_t(1),
                            true, uint32_t(1), uint32_t(1), std::string("softmax"), std::string("greedy"), false, 1.0f,
                            false, false, TYPE_INVALID, TYPE_I4_GROUP, int(128), false};
    MarlinMoeLayer ok, bf, shortp;
    RuntimeConfig half = rc, bf16 = rc;
    half.inter_data_type = TYPE_FP16;
    bf16.inter_data_type = TYPE_BF16;
    expect(ok.Init(p, half, context, 0).OK(), "marlin moe fp16 init");
    expect(ok.GetWorkspaceSize() > 0, "marlin moe workspace size");
    expect(!bf.Init(p, bf16, context, 0).OK(), "marlin moe rejects bf16");
    p.pop_back();
    expect(!shortp.Init(p, half, context, 0).OK(), "marlin moe rejects a short parameter list");
  }
  // moe: fp8 experts / impossible expert groups rejected, int4 and grouped routing accepted
  {
    MoeLayer a, b, c;
    // (a raw parameter vector on purpose: these are checks of what Init itself refuses)
    std::vector<std::any> p{MoeScaleNormMode::NO_NORM, size_t(64), int(0), size_t(8), size_t(256), size_t(256), size_t(2),
                            size_t(1), true, uint32_t(1), uint32_t(1), std::string("softmax"), std::string("greedy"), false,
                            1.0f, false, false, TYPE_INVALID, TYPE_UINT4x2, int(128), false};
    expect(a.Init(p, rc, context, 0).OK(), "moe int4 init");
    expect(a.GetWorkspaceSize() > 0, "moe workspace size");
    auto q = p;
    q[17] = TYPE_FP8_E4M3;
    expect(!b.Init(q, rc, context, 0).OK(), "per-tensor fp8 experts are rejected");
    MoeLayer b2, b3;
    q[17] = TYPE_BLOCK_FP8_E4M3;
    expect(!b2.Init(q, rc, context, 0).OK(), "int4 weights with fp8 activations are rejected");
    q[18] = TYPE_INVALID;
    expect(b3.Init(q, rc, context, 0).OK(), "block-fp8 experts init");
    expect(b3.GetWorkspaceSize() > 0 && b3.BlockM(4096) == 256 && b3.BlockM(64) == 128 && b3.BlockM(32) == 32, "block-fp8 workspace and block size");
    auto r = p;
    r[9] = uint32_t(4);   // 4 groups of 2 experts, 2 kept: top-2 fits
    r[10] = uint32_t(2);
    r[11] = std::string("sigmoid");
    expect(c.Init(r, rc, context, 0).OK(), "grouped sigmoid routing init");
    MoeLayer d, e, f;
    r[9] = uint32_t(3);
    expect(!d.Init(r, rc, context, 0).OK(), "groups that do not divide the experts are rejected");
    r[9] = uint32_t(8);   // groups of one expert, 1 kept: top-2 does not fit
    r[10] = uint32_t(1);
    expect(!e.Init(r, rc, context, 0).OK(), "kept groups smaller than topk are rejected");
    r = p;
    r[11] = std::string("tanh");
    expect(!f.Init(r, rc, context, 0).OK(), "unknown scoring function is rejected");
    expect(ksq_moe_block_m(8 * 2, 8) == 16 && ksq_moe_block_m(64 * 2, 8) == 32 && ksq_moe_block_m(1024 * 8, 256) == 32 && ksq_moe_block_m(2048 * 8, 256) == 256 && ksq_moe_block_m(4096 * 8, 256) == 256,
           "block_m thresholds");
  }
  // the Auto factories: what they derive and what they refuse
  {
    ModelConfig m2;
    m2.is_quant = true;
    m2.quant_config.method = QUANT_GPTQ;
    m2.hidden_units = 4096;
    m2.inter_size = 14336;
    m2.head_num = 32;
    m2.num_key_value_heads = 8;
    m2.size_per_head = 128;
    RuntimeConfig r2 = rc;
    r2.parallel_basic_config.tensor_parallel_size = 2;
    r2.parallel_basic_config.attn_tensor_parallel_size = 2;
    MatMulLayerFactory f2(m2, r2, 0, context);
    size_t k = 0, n = 0;
    bool k_full = false;
    expect(f2.ProjectionShape("model.layers.7.mlp.down_proj.weight", &k, &n, &k_full) && k == 7168 && n == 4096 && !k_full,
           "down_proj: K is the rank's slice");
    expect(f2.ProjectionShape("model.layers.7.mlp.gate_proj.weight", &k, &n, &k_full) && k == 4096 && n == 7168 && k_full,
           "gate_proj: N is the rank's slice");
    expect(f2.ProjectionShape("model.layers.7.self_attn.query_key_value.weight", &k, &n, &k_full) && k == 4096 &&
               n == 128 * (32 + 16) / 2 && k_full, "fused qkv");
    expect(f2.ProjectionShape("model.layers.7.self_attn.o_proj.weight", &k, &n, &k_full) && k == 2048 && n == 4096 && !k_full,
           "o_proj");
    expect(!f2.ProjectionShape("lm_head.weight", &k, &n, &k_full), "a name that is no projection");
    auto weights = std::make_shared<TestWeights>();
    static char placeholder[16];  // shapes and dtypes are all the factories read: no device memory behind these
    weights->weights["lm_head.weight"] = Tensor(MemoryLocation::LOCATION_DEVICE, TYPE_FP16, {16, 16}, 0, placeholder);
    expect(throws([&] { f2.AutoCreateLayer(weights, "lm_head.weight", TYPE_FP16, TYPE_FP16, TYPE_FP16, CUTLASS_LINEAR_BACKEND, {}); }),
           "an unquantized weight has no layer here");
    ModelConfig m3;
    m3.is_quant = true;
    m3.quant_config.method = QUANT_GPTQ;
    m3.hidden_units = 256;
    m3.moe_config.num_experts = 8;
    m3.moe_config.experts_topk = 2;
    m3.moe_config.moe_inter_size = 128;
    m3.moe_config.use_vllm_moe = true;
    MoeLayerFactory f3(m3, rc, 0, context);
    weights->weights["up"] = Tensor(MemoryLocation::LOCATION_DEVICE, TYPE_UINT8, {8, 256, 128}, 0, placeholder);
    weights->weights["down"] = Tensor(MemoryLocation::LOCATION_DEVICE, TYPE_UINT8, {8, 256, 64}, 0, placeholder);
    weights->weights["down7"] = Tensor(MemoryLocation::LOCATION_DEVICE, TYPE_UINT8, {7, 256, 64}, 0, placeholder);
    weights->weights["down_h"] = Tensor(MemoryLocation::LOCATION_DEVICE, TYPE_UINT8, {8, 512, 64}, 0, placeholder);
    expect(f3.AutoCreateMoeLayer(weights, {"up", "down"}, TYPE_UINT8, TYPE_BF16, TYPE_BF16, 0, {MoeScaleNormMode::NO_NORM}) != nullptr,
           "int4 experts through the auto factory");
    expect(throws([&] { f3.AutoCreateMoeLayer(weights, {"up", "down7"}, TYPE_UINT8, TYPE_BF16, TYPE_BF16, 0, {MoeScaleNormMode::NO_NORM}); }),
           "expert counts that differ are refused");
    expect(throws([&] { f3.AutoCreateMoeLayer(weights, {"up", "down_h"}, TYPE_UINT8, TYPE_BF16, TYPE_BF16, 0, {MoeScaleNormMode::NO_NORM}); }),
           "hidden sizes that differ are refused");
  }
  std::printf(failures ? "layer errors: %d FAILED\n" : "layer errors: OK\n", failures);
  return failures ? 1 : 0;
}

int main(int argc, char** argv) {
  if (argc < 2) return 2;
  const std::string mode = argv[1];
  try {
    if (mode == "w4a16") return RunW4A16(argc, argv);
    if (mode == "blockwise") return RunBlockwise(argc, argv);
    if (mode == "fp8_tensor") return RunFp8Tensor(argc, argv);
    if (mode == "moe") return RunMoe(argc, argv);
    if (mode == "moe_fp8") return RunMoeFp8(argc, argv);
    if (mode == "marlin_moe") return RunMarlinMoe(argc, argv);
    if (mode == "w4a8") return RunW4A8(argc, argv);
    if (mode == "errors") return RunErrors();
  } catch (const std::exception& e) {
    std::fprintf(stderr, "exception: %s\n", e.what());
    return 4;
  }
  return 2;
}
