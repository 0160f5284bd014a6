#include "quant_weight_repack.h"

#include <algorithm>
#include <cstring>
#include <vector>

namespace ksana_llm {

namespace {

// Act-order weight of which this rank holds a K range: `groups` are the checkpoint-wide group numbers of its K rows,
// `scales` [G_total, N] the scales of all groups.  Sorted by group, the runs of equal group have arbitrary lengths: each
// run is padded to a multiple of 32 rows (padding rows: index -1, code 8, no contribution) and the whole to a multiple of
// 128, and the scale table gets one row per 32 packed rows, so that the group-32 kernels apply the scales by position.
Tensor PackActOrderSlice(const Tensor& qweight, const Tensor& scales, const std::vector<int32_t>& groups, size_t K, size_t N,
                         int rank, hipStream_t stream) {
  const char* who = "PackGroupQuantWeight";
  const size_t G_total = scales.shape[0];
  std::vector<int32_t> order(K);
  for (size_t i = 0; i < K; ++i) order[i] = static_cast<int32_t>(i);
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return groups[a] < groups[b]; });
  std::vector<int32_t> rows, sorted, block_group;
  rows.reserve(K + K / 4);
  for (size_t i = 0; i < K;) {
    const int32_t g = groups[order[i]];
    if (g < 0 || static_cast<size_t>(g) >= G_total) KLLM_THROW("PackGroupQuantWeight: g_idx names a group the scales do not hold");
    size_t j = i;
    while (j < K && groups[order[j]] == g) rows.push_back(order[j++]);
    while (rows.size() % 32 != 0) rows.push_back(-1);
    sorted.resize(rows.size(), g);
    block_group.resize(rows.size() / 32, g);
    i = j;
  }
  while (rows.size() % 128 != 0) {
    rows.push_back(-1);
    sorted.push_back(sorted.back());
    if (rows.size() % 32 == 0) block_group.push_back(block_group.back());
  }
  const size_t Kp = rows.size();
  Tensor packed(MemoryLocation::LOCATION_DEVICE, TYPE_I4_GROUP, {Kp, N / 2}, rank);
  packed.perm = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_INT32, std::vector<size_t>{Kp}, rank);
  packed.g_idx = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_INT32, std::vector<size_t>{Kp}, rank);
  if (hipMemcpy(packed.perm->GetPtr<void>(), rows.data(), Kp * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess ||
      hipMemcpy(packed.g_idx->GetPtr<void>(), sorted.data(), Kp * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess) {
    KLLM_THROW("PackGroupQuantWeight: cannot upload perm");
  }
  KsqCheck(ksq_w4a16_repack_rows(qweight.GetPtr<void>(), packed.perm->GetPtr<void>(), packed.GetPtr<void>(), K, Kp, N, stream), who);
  // scale row of every 32 packed rows, then the packed scale layout for group size 32.  The table is expanded on the
  // host (one copy down, one up: a device copy per 32 packed rows would be more than a thousand tiny copies per weight)
  const size_t row_bytes = N * GetTypeSize(scales.dtype);
  Tensor expanded(MemoryLocation::LOCATION_DEVICE, scales.dtype, {Kp / 32, N}, rank);
  {
    const size_t table_rows = scales.shape[0];
    std::vector<char> table(table_rows * row_bytes), wide((Kp / 32) * row_bytes);
    if (hipStreamSynchronize(stream) != hipSuccess ||
        hipMemcpy(table.data(), scales.GetPtr<void>(), table.size(), hipMemcpyDeviceToHost) != hipSuccess) {
      KLLM_THROW("PackGroupQuantWeight: cannot read the scales");
    }
    for (size_t b = 0; b < Kp / 32; ++b) {
      const size_t g = static_cast<size_t>(block_group[b]);
      if (g >= table_rows) KLLM_THROW("PackGroupQuantWeight: g_idx names a group the scales do not hold");
      std::memcpy(wide.data() + b * row_bytes, table.data() + g * row_bytes, row_bytes);
    }
    if (hipMemcpy(expanded.GetPtr<void>(), wide.data(), wide.size(), hipMemcpyHostToDevice) != hipSuccess) {
      KLLM_THROW("PackGroupQuantWeight: cannot upload the expanded scales");
    }
  }
  packed.scales = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, scales.dtype, std::vector<size_t>{Kp / 32, N}, rank);
  KsqCheck(ksq_w4a16_repack_scales(expanded.GetPtr<void>(), KSQ_SCALE_GN, packed.scales->GetPtr<void>(), 1, Kp, N, 32,
                                   KsqDtype(scales.dtype, who), stream), who);
  if (hipStreamSynchronize(stream) != hipSuccess) KLLM_THROW("PackGroupQuantWeight: stream error");  // `expanded` dies here
  return packed;
}

}  // namespace

Tensor PackGroupQuantWeight(const Tensor& qweight, const Tensor& scales, const Tensor* qzeros, QuantMode method,
                            size_t group_size, int rank, hipStream_t stream, const Tensor* g_idx, bool k_full) {
  const char* who = "PackGroupQuantWeight";
  if (method != QUANT_GPTQ && method != QUANT_AWQ) KLLM_THROW("PackGroupQuantWeight: method must be GPTQ or AWQ");
  if (qweight.shape.size() != 2 || scales.shape.size() != 2) KLLM_THROW("PackGroupQuantWeight: 2-D tensors expected");
  const bool awq = method == QUANT_AWQ;
  const size_t K = awq ? qweight.shape[0] : qweight.shape[0] * 8;
  const size_t N = awq ? qweight.shape[1] * 8 : qweight.shape[1];
  const bool k_slice = g_idx != nullptr && !k_full;  // the scales then cover the whole checkpoint's groups
  if ((!k_slice && scales.shape[0] * group_size != K) || scales.shape[1] != N) KLLM_THROW("PackGroupQuantWeight: scales shape mismatch");
  if (awq && !qzeros) KLLM_THROW("PackGroupQuantWeight: AWQ needs qzeros");
  const int dtype = KsqDtype(scales.dtype, who);

  if (k_slice) {
    if (awq) KLLM_THROW("PackGroupQuantWeight: g_idx (act-order) belongs to GPTQ checkpoints");
    // padding rows take code 8, which is nothing only under the symmetric zero point
    if (qzeros) KLLM_THROW("PackGroupQuantWeight: a K range of an act-order weight is packed for symmetric GPTQ only (qzeros given)");
    if (g_idx->GetElementNumber() != K) KLLM_THROW("PackGroupQuantWeight: g_idx must have K entries");
    std::vector<int32_t> groups(K);
    if (hipStreamSynchronize(stream) != hipSuccess ||
        hipMemcpy(groups.data(), g_idx->GetPtr<void>(), K * sizeof(int32_t), hipMemcpyDeviceToHost) != hipSuccess) {
      KLLM_THROW("PackGroupQuantWeight: cannot read g_idx");
    }
    return PackActOrderSlice(qweight, scales, groups, K, N, rank, stream);
  }
  Tensor packed(MemoryLocation::LOCATION_DEVICE, TYPE_I4_GROUP, {K, N / 2}, rank);
  if (g_idx) {
    if (awq) KLLM_THROW("PackGroupQuantWeight: g_idx (act-order) belongs to GPTQ checkpoints");
    if (g_idx->GetElementNumber() != K) KLLM_THROW("PackGroupQuantWeight: g_idx must have K entries");
    std::vector<int32_t> groups(K), perm(K);
    if (hipStreamSynchronize(stream) != hipSuccess ||
        hipMemcpy(groups.data(), g_idx->GetPtr<void>(), K * sizeof(int32_t), hipMemcpyDeviceToHost) != hipSuccess) {
      KLLM_THROW("PackGroupQuantWeight: cannot read g_idx");
    }
    for (size_t i = 0; i < K; ++i) perm[i] = static_cast<int32_t>(i);
    std::stable_sort(perm.begin(), perm.end(), [&](int32_t a, int32_t b) { return groups[a] < groups[b]; });
    std::vector<int32_t> sorted(K);
    for (size_t i = 0; i < K; ++i) {
      sorted[i] = groups[perm[i]];
      // sorted, every group must cover exactly its group_size rows: only then do the scales apply by position
      if (sorted[i] != static_cast<int32_t>(i / group_size)) KLLM_THROW("PackGroupQuantWeight: g_idx does not hold group_size rows per group");
    }
    packed.perm = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_INT32, std::vector<size_t>{K}, rank);
    packed.g_idx = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_INT32, std::vector<size_t>{K}, rank);
    if (hipMemcpy(packed.perm->GetPtr<void>(), perm.data(), K * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(packed.g_idx->GetPtr<void>(), sorted.data(), K * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess) {
      KLLM_THROW("PackGroupQuantWeight: cannot upload perm");
    }
    KsqCheck(ksq_w4a16_repack_act_order(qweight.GetPtr<void>(), packed.perm->GetPtr<void>(), packed.GetPtr<void>(), K, N, stream), who);
  } else {
    KsqCheck(ksq_w4a16_repack(qweight.GetPtr<void>(), awq ? KSQ_SRC_AWQ : KSQ_SRC_GPTQ, packed.GetPtr<void>(), 1, K, N, stream), who);
  }
  packed.scales = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, scales.dtype, scales.shape, rank);
  KsqCheck(ksq_w4a16_repack_scales(scales.GetPtr<void>(), KSQ_SCALE_GN, packed.scales->GetPtr<void>(), 1, K, N, group_size, dtype, stream), who);
  if (awq) {
    packed.zeros = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_UINT8, std::vector<size_t>{K / group_size, N}, rank);
    KsqCheck(ksq_w4a16_repack_zeros(qzeros->GetPtr<void>(), KSQ_ZERO_AWQ_PACKED, packed.zeros->GetPtr<void>(), K, N, group_size, stream), who);
  }
  return packed;
}

Tensor PackGptqExpertWeight(const Tensor& qweight, const Tensor& scales, size_t group_size, int rank, hipStream_t stream,
                            const Tensor* g_idx) {
  const char* who = "PackGptqExpertWeight";
  if (qweight.shape.size() != 3 || scales.shape.size() != 3) KLLM_THROW("PackGptqExpertWeight: 3-D tensors expected");
  const size_t E = qweight.shape[0], K = qweight.shape[1] * 8, N = qweight.shape[2];
  if (scales.shape[0] != E || scales.shape[1] * group_size != K || scales.shape[2] != N) {
    KLLM_THROW("PackGptqExpertWeight: scales shape mismatch");
  }
  const int dtype = KsqDtype(scales.dtype, who);
  Tensor packed(MemoryLocation::LOCATION_DEVICE, TYPE_INT32, {E, K / 16, 2 * N}, rank);
  if (g_idx) {
    // act-order: every expert has its own group index; its rows are sorted by group (stable), as MarlinSortGIdx and the
    // perm form of gptq_marlin_repack do per expert, and the layer gathers the activation columns through `perm`
    if (g_idx->GetElementNumber() != E * K) KLLM_THROW("PackGptqExpertWeight: g_idx must have E * K entries");
    std::vector<int32_t> groups(E * K), perm(E * K), sorted(E * K);
    if (hipStreamSynchronize(stream) != hipSuccess ||
        hipMemcpy(groups.data(), g_idx->GetPtr<void>(), E * K * sizeof(int32_t), hipMemcpyDeviceToHost) != hipSuccess) {
      KLLM_THROW("PackGptqExpertWeight: cannot read g_idx");
    }
    for (size_t e = 0; e < E; ++e) {
      int32_t* pe = perm.data() + e * K;
      const int32_t* ge = groups.data() + e * K;
      for (size_t i = 0; i < K; ++i) pe[i] = static_cast<int32_t>(i);
      std::stable_sort(pe, pe + K, [&](int32_t a, int32_t b) { return ge[a] < ge[b]; });
      for (size_t i = 0; i < K; ++i) {
        sorted[e * K + i] = ge[pe[i]];
        if (sorted[e * K + i] != static_cast<int32_t>(i / group_size))
          KLLM_THROW("PackGptqExpertWeight: g_idx does not hold group_size rows per group");
      }
    }
    packed.perm = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_INT32, std::vector<size_t>{E, K}, rank);
    packed.g_idx = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, TYPE_INT32, std::vector<size_t>{E, K}, rank);
    if (hipMemcpy(packed.perm->GetPtr<void>(), perm.data(), E * K * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(packed.g_idx->GetPtr<void>(), sorted.data(), E * K * sizeof(int32_t), hipMemcpyHostToDevice) != hipSuccess) {
      KLLM_THROW("PackGptqExpertWeight: cannot upload perm");
    }
    for (size_t e = 0; e < E; ++e) {
      KsqCheck(ksq_w4a16_repack_act_order(qweight.GetPtr<int32_t>() + e * (K / 8) * N, packed.perm->GetPtr<int32_t>() + e * K,
                                          packed.GetPtr<char>() + e * (K * N / 2), K, N, stream),
               who);
    }
  } else {
    KsqCheck(ksq_w4a16_repack(qweight.GetPtr<void>(), KSQ_SRC_GPTQ, packed.GetPtr<void>(), E, K, N, stream), who);
  }
  packed.scales = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, scales.dtype, scales.shape, rank);
  KsqCheck(ksq_w4a16_repack_scales(scales.GetPtr<void>(), KSQ_SCALE_GN, packed.scales->GetPtr<void>(), E, K, N, group_size, dtype, stream), who);
  return packed;
}

Tensor PackMoeExpertWeight(const Tensor& experts, const Tensor& scales, size_t group_size, int rank, hipStream_t stream) {
  const char* who = "PackMoeExpertWeight";
  if (experts.shape.size() != 3 || scales.shape.size() != 3) KLLM_THROW("PackMoeExpertWeight: 3-D tensors expected");
  const size_t E = experts.shape[0], N = experts.shape[1], K = experts.shape[2] * 2;
  if (scales.shape[0] != E || scales.shape[1] != N || scales.shape[2] * group_size != K) {
    KLLM_THROW("PackMoeExpertWeight: scales shape mismatch");
  }
  const int dtype = KsqDtype(scales.dtype, who);
  Tensor packed(MemoryLocation::LOCATION_DEVICE, TYPE_UINT8, experts.shape, rank);
  KsqCheck(ksq_w4a16_repack(experts.GetPtr<void>(), KSQ_SRC_MOE_NK, packed.GetPtr<void>(), E, K, N, stream), who);
  packed.scales = std::make_shared<Tensor>(MemoryLocation::LOCATION_DEVICE, scales.dtype, scales.shape, rank);
  KsqCheck(ksq_w4a16_repack_scales(scales.GetPtr<void>(), KSQ_SCALE_NG, packed.scales->GetPtr<void>(), E, K, N, group_size, dtype, stream), who);
  return packed;
}

Tensor PackFp8Weight(const Tensor& weight, int rank, hipStream_t stream) {
  const char* who = "PackFp8Weight";
  if (weight.dtype != TYPE_FP8_E4M3) KLLM_THROW("PackFp8Weight: weight must be TYPE_FP8_E4M3");
  if (weight.shape.size() != 2 && weight.shape.size() != 3) KLLM_THROW("PackFp8Weight: [N, K] or [E, N, K] expected");
  const size_t E = weight.shape.size() == 3 ? weight.shape[0] : 1;
  const size_t N = weight.shape[weight.shape.size() - 2], K = weight.shape.back();
  Tensor packed(MemoryLocation::LOCATION_DEVICE, TYPE_FP8_E4M3, weight.shape, rank);
  KsqCheck(ksq_fp8_repack_weight(weight.GetPtr<void>(), packed.GetPtr<void>(), E, N, K, stream), who);
  packed.scales = weight.scales;
  packed.zeros = weight.zeros;
  packed.input_scales = weight.input_scales;
  packed.weight_scales = weight.weight_scales;
  packed.pre_quant_scales = weight.pre_quant_scales;
  packed.input_alpha = weight.input_alpha;
  return packed;
}

Tensor PackW4A8Weight(const Tensor& weight, int rank, hipStream_t stream) {
  const char* who = "PackW4A8Weight";
  if (weight.shape.size() != 2) KLLM_THROW("PackW4A8Weight: [K, N/2] expected");
  if (GetTypeSize(weight.dtype) != 1) KLLM_THROW("PackW4A8Weight: one byte per two weights expected");
  const size_t K = weight.shape[0], N = 2 * weight.shape[1];
  Tensor packed(MemoryLocation::LOCATION_DEVICE, weight.dtype, weight.shape, rank);
  KsqCheck(ksq_w4a8_repack_weight(weight.GetPtr<void>(), packed.GetPtr<void>(), N, K, stream), who);
  packed.input_scales = weight.input_scales;
  packed.weight_scales = weight.weight_scales;
  packed.pre_quant_scales = weight.pre_quant_scales;
  packed.input_alpha = weight.input_alpha;
  packed.alpha = weight.alpha;
  return packed;
}

}  // namespace ksana_llm
