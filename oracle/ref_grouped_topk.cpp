// Test infrastructure, not product code.  C entry point around the reference's own host implementation of the
// DeepSeek-V3 grouped top-k router (3rdparty/LLM_kernels/tests/references/deepseek_v3_grouped_topk.h:134-227,
// RunDeepSeekV3GroupedTopkRef), the one source file of the quantized-GEMM / MoE path that compiles with g++ alone.  The
// header is included from the reference tree where it lies (make -C oracle ref REF=/root/reference); nothing of it is
// copied here.  It takes fp32 logits and an fp32 correction bias, scores with sigmoid, ranks groups by their top-2 sum
// and always renormalizes: the checks that use it stay inside that case.
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstddef>

#include "tests/references/deepseek_v3_grouped_topk.h"

extern "C" __attribute__((visibility("default"))) void ksq_ref_grouped_topk(
    const float* gating, const float* e_bias, float routed_scaling_factor, float* topk_weights, int32_t* topk_ids,
    int tokens, int experts, int topk, int num_expert_group, int topk_group) {
  llm_kernels::nvidia::test::RunDeepSeekV3GroupedTopkRef<float>(
      const_cast<float*>(gating), const_cast<float*>(e_bias), routed_scaling_factor, topk_weights, topk_ids, tokens,
      experts, topk, num_expert_group, topk_group);
}
