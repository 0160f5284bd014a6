"""C++ layer classes (ksanallm_amd/layers) driven through their factories by tests/cpp/layer_test.

The driver follows the call order model code uses - factory CreateLayer -> Init -> GetWorkspaceSize ->
SetWorkspaceBuffer -> Preprocess -> Forward - on raw tensors written here, and its output is compared with the CPU
oracle under the GEMM tolerance (rel-L2 <= 5e-3, max-abs <= 2e-2).  The error-behaviour checks need no GPU.
"""
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "tests", "cpp", "layer_test")
TNAME = {H.F16: "f16", H.BF16: "bf16"}


def run_driver(*args):
    if not os.path.exists(DRIVER):
        pytest.fail("tests/cpp/layer_test is not built: run `python -m ksanallm_amd.build`")
    r = subprocess.run([DRIVER] + [str(a) for a in args], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, "layer_test %s -> rc %d\n%s\n%s" % (" ".join(map(str, args)), r.returncode, r.stdout, r.stderr)
    return r.stdout


def read_out(path, dtype, shape):
    bits = np.fromfile(path, dtype=np.uint16).reshape(shape)
    return torch.from_numpy(bits.view(np.int16)).view(H.TORCH_DT[dtype])


def test_layer_error_behaviour():
    assert "layer errors: OK" in run_driver("errors")


@pytest.mark.gpu
@pytest.mark.parametrize("method,dtype,backend,m,n,k,group", [
    ("gptq", H.F16, "marlin", 1, 512, 1024, 128),
    ("gptq", H.BF16, "machete", 16, 1024, 512, 128),
    ("awq", H.F16, "cutlass", 4, 768, 1024, 128),
    ("awq", H.BF16, "machete", 33, 512, 2048, 64),
    ("awq", H.BF16, "cutlass", 192, 1024, 1024, 128),
])
def test_w4a16_layers(tmp_path, method, dtype, backend, m, n, k, group):
    d = H.make_w4a16(9000 + m + n, m, n, k, group, dtype, method == "awq")
    d["qweight"].numpy().tofile(tmp_path / "qweight.bin")
    H.bits_of(d["scales"]).tofile(tmp_path / "scales.bin")
    H.bits_of(d["x"]).tofile(tmp_path / "x.bin")
    if method == "awq":
        d["qzeros"].numpy().tofile(tmp_path / "qzeros.bin")
    run_driver("w4a16", tmp_path, method, TNAME[dtype], backend, m, n, k, group)
    y = read_out(tmp_path / "y.bin", dtype, (m, n))
    H.check_gemm(y, H.w4a16_oracle(d), dtype, "%s %s layer" % (backend, method), weights_rounded=m > 32)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,backend,m,n,k", [(H.F16, "marlin", 3, 512, 1024), (H.BF16, "machete", 100, 1024, 512)])
def test_w4a16_layer_act_order(tmp_path, oracle, dtype, backend, m, n, k):
    d = H.make_w4a16(9050 + m, m, n, k, 128, dtype, False)
    g_idx = (torch.randperm(k, generator=H.gen(9060 + k)) // 128).to(torch.int32)
    d["qweight"].numpy().tofile(tmp_path / "qweight.bin")
    H.bits_of(d["scales"]).tofile(tmp_path / "scales.bin")
    H.bits_of(d["x"]).tofile(tmp_path / "x.bin")
    g_idx.numpy().tofile(tmp_path / "g_idx.bin")
    run_driver("w4a16", tmp_path, "gptq", TNAME[dtype], backend, m, n, k, 128, 1)
    y = read_out(tmp_path / "y.bin", dtype, (m, n))
    ref = oracle.gptq_act_order_gemm(H.bits_of(d["x"]), d["codes"], H.bits_of(d["scales"]), g_idx.numpy(), dtype)
    H.check_gemm(y, ref, dtype, "%s act-order layer" % backend, weights_rounded=m > 32)


@pytest.mark.gpu
@pytest.mark.parametrize("context_tp", [2, 1])   # 1: the context reports fewer ranks than the cut the factory applied
@pytest.mark.parametrize("dtype,backend,m,n,k", [(H.F16, "marlin", 3, 512, 1024), (H.BF16, "marlin", 40, 256, 1536)])
def test_w4a16_layer_act_order_k_range(tmp_path, oracle, dtype, backend, m, n, k, context_tp):
    """is_k_full = false: this rank holds rows [0, k) of an act-order checkpoint with 2k rows (mlp.down_proj under two
    tensor-parallel ranks).  Its rows belong to arbitrary groups of the whole checkpoint; the oracle is the definition
    y = x . ((code - 8) * scale[g_idx[row]]) over the rank's rows."""
    g = H.gen(9070 + k)
    full = H.make_w4a16(9071 + m, m, n, 2 * k, 128, dtype, False)         # the whole checkpoint: codes, scales of all groups
    g_idx_full = (torch.randperm(2 * k, generator=g) // 128).to(torch.int32)
    codes, g_idx = full["codes"][:k], g_idx_full[:k].contiguous()
    x = full["x"][:, :k].contiguous()
    torch.from_numpy(oracle.gptq_pack(codes).view(np.int32)).numpy().tofile(tmp_path / "qweight.bin")
    H.bits_of(full["scales"]).tofile(tmp_path / "scales.bin")
    H.bits_of(x).tofile(tmp_path / "x.bin")
    g_idx.numpy().tofile(tmp_path / "g_idx.bin")
    run_driver("w4a16", tmp_path, "gptq", TNAME[dtype], backend, m, n, k, 128, 1, 1, context_tp)
    y = read_out(tmp_path / "y.bin", dtype, (m, n))
    ref = oracle.gptq_act_order_gemm(H.bits_of(x), codes, H.bits_of(full["scales"]), g_idx.numpy(), dtype)
    H.check_gemm(y, ref, dtype, "%s act-order K-range layer" % backend, weights_rounded=m > 32)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,m,n,k,fuse,max_m", [(H.BF16, 5, 512, 1024, 0, None), (H.F16, 33, 256, 512, 0, None),
                                                    (H.BF16, 16, 512, 1024, 1, None),
                                                    # odd max_m with K cut over workgroups: the GEMM's scratch behind
                                                    # a_q and a_s must still start on an aligned address
                                                    (H.BF16, 37, 256, 1664, 0, 37), (H.BF16, 35, 256, 640, 0, 41)])
def test_blockwise_layer(tmp_path, oracle, dtype, m, n, k, fuse, max_m):
    g = H.gen(9100 + m)
    w = (torch.randn((n, k), generator=g) * 0.02).to(torch.bfloat16).float().numpy()
    bq, bs = oracle.fp8_block_quant_weight(w)
    x = (torch.randn((m, 2 * k if fuse else k), generator=g)).to(H.TORCH_DT[dtype])
    bq.tofile(tmp_path / "w.bin")
    bs.astype(np.float32).tofile(tmp_path / "w_scale.bin")
    H.bits_of(x).tofile(tmp_path / "x.bin")
    run_driver("blockwise", tmp_path, TNAME[dtype], m, n, k, fuse, *([] if max_m is None else [max_m]))
    y = read_out(tmp_path / "y.bin", dtype, (m, n))
    q, s = oracle.fp8_group_quant(H.bits_of(x), k, 128, True, bool(fuse), dtype)
    ref = oracle.fp8_blockwise_gemm(q, s, bq, bs, True)
    # the fused silu*mul may differ from the oracle by one rounding of T before quantization: compare as a GEMM
    H.check_gemm(y, ref, dtype, "blockwise layer")


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(5, 512, 1024), (70, 256, 640)])
def test_blockwise_layer_fp32_activations(tmp_path, oracle, m, n, k):
    """inter_data_type TYPE_FP32 (DISPATCH_BY_3_DTYPE in the reference's Forward): fp32 in, fp32 out."""
    g = H.gen(9150 + m)
    w = (torch.randn((n, k), generator=g) * 0.02).to(torch.bfloat16).float().numpy()
    bq, bs = oracle.fp8_block_quant_weight(w)
    x = torch.randn((m, k), generator=g)
    bq.tofile(tmp_path / "w.bin")
    bs.astype(np.float32).tofile(tmp_path / "w_scale.bin")
    x.numpy().tofile(tmp_path / "x.bin")
    run_driver("blockwise", tmp_path, "f32", m, n, k, 0)
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32).reshape(m, n)
    q, s = oracle.fp8_group_quant(x.numpy(), k, 128, True, False, oracle.F32)
    ref = oracle.fp8_blockwise_gemm(q, s, bq, bs, True)
    H.check_gemm_f32(torch.from_numpy(y), ref, "blockwise layer fp32")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tokens,renorm,scaling,routing", [
    (H.BF16, 1, 0, 2.5, None), (H.F16, 24, 1, 1.0, None), (H.BF16, 70, 0, 1.0, None), (H.BF16, 400, 0, 1.0, None),
    # 2: scale-norm mode RE_NORM with norm_topk_prob false - the routers follow norm_topk_prob alone (no renormalization)
    (H.BF16, 24, 2, 1.0, None),
    # DeepSeek-V3 style routing: 4 groups of 4 experts, 2 kept, sigmoid scores with a correction bias (layer input 5)
    (H.BF16, 33, 1, 2.5, (4, 2, "sigmoid", True)), (H.F16, 5, 0, 1.0, (2, 1, "softmax", False))])
def test_moe_layer(tmp_path, oracle, dtype, tokens, renorm, scaling, routing):
    E, hidden, inter, topk = 16, 256, 128, 4
    g = H.gen(9200 + tokens)
    w13 = torch.randint(0, 256, (E, 2 * inter, hidden // 2), generator=g, dtype=torch.uint8)
    w2 = torch.randint(0, 256, (E, hidden, inter // 2), generator=g, dtype=torch.uint8)
    s13 = H.uniform(g, (E, 2 * inter, hidden // 128), 0.002, 0.01, dtype)
    s2 = H.uniform(g, (E, hidden, inter // 128), 0.002, 0.01, dtype)
    x = torch.randn((tokens, hidden), generator=g).to(H.TORCH_DT[dtype])
    gating = torch.randn((tokens, E), generator=g)
    for name, arr in (("w13", w13.numpy()), ("w2", w2.numpy()), ("s13", H.bits_of(s13)), ("s2", H.bits_of(s2)),
                      ("x", H.bits_of(x)), ("gating", gating.numpy())):
        arr.tofile(tmp_path / (name + ".bin"))
    if routing is None:
        run_driver("moe", tmp_path, TNAME[dtype], tokens, E, hidden, inter, topk, renorm, scaling)
        tw, ids = oracle.moe_topk_softmax(gating.numpy(), topk, renorm == 1, scaling, 2)
    else:
        groups, topk_group, scoring, use_bias = routing
        bias = (torch.rand(E, generator=g) * 0.2 - 0.1) if use_bias else None
        if use_bias:
            bias.numpy().tofile(tmp_path / "bias.bin")
        run_driver("moe", tmp_path, TNAME[dtype], tokens, E, hidden, inter, topk, renorm, scaling, groups, topk_group,
                   scoring, int(use_bias))
        tw, ids = oracle.moe_grouped_topk(gating.numpy(), None if bias is None else bias.numpy(), topk, groups,
                                          topk_group, scoring == "sigmoid", renorm == 1, scaling, 2)
    y = read_out(tmp_path / "y.bin", dtype, (tokens, hidden))
    ref = oracle.moe_forward(H.bits_of(x), w13.numpy(), H.bits_of(s13), w2.numpy(), H.bits_of(s2), ids, tw, 128, dtype)
    ref = oracle.from_bits(ref, dtype)
    # from 40 rows per expert on both GEMMs run through the MFMA tile kernel, which rounds the dequantized weights to T:
    # each GEMM on its own is held to 5e-3 (tests/test_gpu_moe.py), two in a row compound to sqrt(2) of that
    rounded = tokens * topk // E >= 40
    H.check_gemm(y, ref, dtype, "moe layer", weights_rounded=rounded, rel_l2_max=5e-3 * (2 ** 0.5 if rounded else 1.0))


# GPTQ experts behind the Marlin MoE interface: checkpoint-layout int32 words, fp16 gating output, plain softmax router
@pytest.mark.gpu
@pytest.mark.parametrize("tokens,renorm", [(1, 0), (37, 1), (400, 1)])
def test_marlin_moe_layer(tmp_path, oracle, tokens, renorm):
    E, hidden, inter, topk = 16, 256, 128, 4
    dtype = H.F16
    g = H.gen(9300 + tokens)

    def experts(n, k):
        codes = torch.randint(0, 16, (E, n, k), generator=g, dtype=torch.uint8).numpy()
        moe_bytes = (codes[:, :, 0::2] | (codes[:, :, 1::2] << 4)).astype(np.uint8)          # [E, n, k/2], low nibble = even k
        c = codes.transpose(0, 2, 1).reshape(E, k // 8, 8, n).astype(np.uint32)              # [E, k/8, 8, n]
        words = np.zeros((E, k // 8, n), np.uint32)
        for j in range(8):
            words |= c[:, :, j, :] << np.uint32(4 * j)                                          # GPTQ: nibble j = row 8i+j
        scales = H.uniform(g, (E, n, k // 128), 0.002, 0.01, dtype)
        return moe_bytes, words.view(np.int32), scales

    w13, qw13, s13 = experts(2 * inter, hidden)
    w2, qw2, s2 = experts(hidden, inter)
    x = torch.randn((tokens, hidden), generator=g).to(H.TORCH_DT[dtype])
    gating = torch.randn((tokens, E), generator=g).to(torch.float16)
    for name, arr in (("qw13", qw13), ("qw2", qw2), ("s13", H.bits_of(s13.transpose(1, 2).contiguous())),
                      ("s2", H.bits_of(s2.transpose(1, 2).contiguous())), ("x", H.bits_of(x)), ("gating", H.bits_of(gating))):
        np.ascontiguousarray(arr).tofile(tmp_path / (name + ".bin"))
    run_driver("marlin_moe", tmp_path, TNAME[dtype], tokens, E, hidden, inter, topk, renorm)
    y = read_out(tmp_path / "y.bin", dtype, (tokens, hidden))
    tw, ids = oracle.moe_topk_softmax(H.bits_of(gating), topk, bool(renorm), 1.0, H.F16)
    ref = oracle.from_bits(oracle.moe_forward(H.bits_of(x), w13, H.bits_of(s13), w2, H.bits_of(s2), ids, tw, 128, dtype), dtype)
    rounded = tokens * topk // E >= 40
    H.check_gemm(y, ref, dtype, "marlin moe layer", weights_rounded=rounded, rel_l2_max=5e-3 * (2 ** 0.5 if rounded else 1.0))


def _act_order_experts(g, E, n, k, dtype):
    """GPTQ act-order expert stack: codes [E, k, n] in checkpoint row order, words [E, k/8, n], scales [E, k/128, n],
    g_idx [E, k] = a random assignment of the k rows to k/128 groups of 128 rows each."""
    codes = torch.randint(0, 16, (E, k, n), generator=g, dtype=torch.uint8).numpy()
    c = codes.reshape(E, k // 8, 8, n).astype(np.uint32)
    words = np.zeros((E, k // 8, n), np.uint32)
    for j in range(8):
        words |= c[:, :, j, :] << np.uint32(4 * j)
    scales = H.uniform(g, (E, k // 128, n), 0.002, 0.01, dtype)
    g_idx = np.stack([(torch.randperm(k, generator=g).numpy() // 128) for _ in range(E)]).astype(np.int32)
    return codes, words.view(np.int32), scales, g_idx


@pytest.mark.gpu
@pytest.mark.parametrize("tokens,renorm", [(1, 0), (9, 1), (200, 1)])
def test_marlin_moe_layer_act_order(tmp_path, oracle, tokens, renorm):
    """Experts quantized with desc_act: every expert has its own g_idx.  The oracle applies the definition
    (scale[g_idx[k]] per row), the layer sorts the rows at load time and gathers the activations per slot."""
    E, hidden, inter, topk = 16, 256, 128, 4
    dtype = H.F16
    g = H.gen(9800 + tokens)
    c13, qw13, s13, g13 = _act_order_experts(g, E, 2 * inter, hidden, dtype)
    c2, qw2, s2, g2 = _act_order_experts(g, E, hidden, inter, dtype)
    x = torch.randn((tokens, hidden), generator=g).to(H.TORCH_DT[dtype])
    gating = torch.randn((tokens, E), generator=g).to(torch.float16)
    for name, arr in (("qw13", qw13), ("qw2", qw2), ("s13", H.bits_of(s13)), ("s2", H.bits_of(s2)), ("g13", g13), ("g2", g2),
                      ("x", H.bits_of(x)), ("gating", H.bits_of(gating))):
        np.ascontiguousarray(arr).tofile(tmp_path / (name + ".bin"))
    run_driver("marlin_moe", tmp_path, TNAME[dtype], tokens, E, hidden, inter, topk, renorm, 1)
    y = read_out(tmp_path / "y.bin", dtype, (tokens, hidden))
    tw, ids = oracle.moe_topk_softmax(H.bits_of(gating), topk, bool(renorm), 1.0, H.F16)
    ref = oracle.from_bits(oracle.moe_act_order_forward(H.bits_of(x), c13, H.bits_of(s13), g13, c2, H.bits_of(s2), g2, ids, tw,
                                                        dtype), dtype)
    rounded = tokens * topk // E >= 40
    H.check_gemm(y, ref, dtype, "marlin moe layer, act-order", weights_rounded=rounded,
                 rel_l2_max=5e-3 * (2 ** 0.5 if rounded else 1.0))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tokens,renorm,scaling", [(H.BF16, 1, 0, 2.5), (H.F16, 40, 1, 1.0), (H.BF16, 300, 1, 1.0)])
def test_moe_layer_block_fp8(tmp_path, oracle, dtype, tokens, renorm, scaling):
    E, hidden, inter, topk = 16, 256, 128, 4
    g = H.gen(9400 + tokens)

    def experts(n, k):
        w = (torch.randn((E, n, k), generator=g) * 0.02).to(torch.bfloat16).float().numpy()
        q = np.empty((E, n, k), np.uint8)
        s = np.empty((E, (n + 127) // 128, k // 128), np.float32)
        for e in range(E):
            q[e], s[e] = oracle.fp8_block_quant_weight(w[e])
        return q, s

    w13, s13 = experts(2 * inter, hidden)
    w2, s2 = experts(hidden, inter)
    x = torch.randn((tokens, hidden), generator=g).to(H.TORCH_DT[dtype])
    gating = torch.randn((tokens, E), generator=g)
    for name, arr in (("w13", w13), ("w2", w2), ("s13", s13), ("s2", s2), ("x", H.bits_of(x)), ("gating", gating.numpy())):
        arr.tofile(tmp_path / (name + ".bin"))
    run_driver("moe_fp8", tmp_path, TNAME[dtype], tokens, E, hidden, inter, topk, renorm, scaling)
    y = read_out(tmp_path / "y.bin", dtype, (tokens, hidden))
    tw, ids = oracle.moe_topk_softmax(gating.numpy(), topk, bool(renorm), scaling, 2)
    ref = oracle.from_bits(oracle.moe_fp8_forward(H.bits_of(x), w13, s13, w2, s2, ids, tw, dtype), dtype)
    # GEMM tolerance, as for the block test in tests/test_gpu_moe.py (the fused silu*mul quantizer is not bit-pinned)
    H.check_gemm(y, ref, dtype, "block-fp8 moe layer")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,m,n,k,static", [(H.BF16, 1, 512, 1024, 0), (H.F16, 77, 2304, 512, 1), (H.BF16, 300, 1024, 2048, 0)])
def test_fp8_per_tensor_layer(tmp_path, oracle, dtype, m, n, k, static):
    g = H.gen(9600 + m)
    w = (torch.randn((n, k), generator=g) * 0.02).to(torch.bfloat16)
    wq, ws = oracle.fp8_channel_quant(H.bits_of(w).reshape(1, -1), H.BF16)
    x = torch.randn((m, k), generator=g).to(H.TORCH_DT[dtype])
    wq.tofile(tmp_path / "w.bin")
    ws.tofile(tmp_path / "w_scale.bin")
    H.bits_of(x).tofile(tmp_path / "x.bin")
    in_scale = np.array([0.012], np.float32)
    in_scale.tofile(tmp_path / "in_scale.bin")
    run_driver("fp8_tensor", tmp_path, TNAME[dtype], m, n, k, static)
    y = read_out(tmp_path / "y.bin", dtype, (m, n))
    xq, xs = oracle.fp8_channel_quant(H.bits_of(x).reshape(1, -1), dtype, scale=in_scale if static else None)
    ref = oracle.fp8_tensor_gemm(xq.reshape(m, k), xs[0], wq.reshape(n, k), ws[0])
    H.check_gemm(y, ref, dtype, "fp8 per-tensor layer")


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,static", [(3, 512, 1024, 0), (77, 256, 512, 1)])
def test_fp8_per_tensor_layer_fp32_activations(tmp_path, oracle, m, n, k, static):
    """inter_data_type TYPE_FP32: fp32 in, fp32 out, as the reference's map registers the layer (matmul_layer_factory.cpp:70)."""
    g = H.gen(9650 + m)
    w = (torch.randn((n, k), generator=g) * 0.02).to(torch.bfloat16)
    wq, ws = oracle.fp8_channel_quant(H.bits_of(w).reshape(1, -1), H.BF16)
    x = torch.randn((m, k), generator=g)
    wq.tofile(tmp_path / "w.bin")
    ws.tofile(tmp_path / "w_scale.bin")
    x.numpy().tofile(tmp_path / "x.bin")
    in_scale = np.array([0.012], np.float32)
    in_scale.tofile(tmp_path / "in_scale.bin")
    run_driver("fp8_tensor", tmp_path, "f32", m, n, k, static)
    y = np.fromfile(tmp_path / "y.bin", dtype=np.float32).reshape(m, n)
    xq, xs = oracle.fp8_channel_quant(x.numpy().reshape(1, -1), oracle.F32, scale=in_scale if static else None)
    ref = oracle.fp8_tensor_gemm(xq.reshape(m, k), xs[0], wq.reshape(n, k), ws[0])
    H.check_gemm_f32(torch.from_numpy(y), ref, "fp8 per-tensor layer fp32")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,m,n,k,per_channel", [(H.BF16, 1, 512, 1024, 0), (H.F16, 77, 2304, 512, 1),
                                                      (H.BF16, 300, 1024, 2048, 1), (H.F16, 20, 48, 128, 0)])
def test_w4a8_layer(tmp_path, oracle, dtype, m, n, k, per_channel):
    """FinegrainedMixedDtypeGemmLayer through the factory: static per-tensor scale, or the per-channel divisor
    input_scale / pre_quant_scale the reference's loader prepares (w4a8_awq_method.cpp:193-200)."""
    g = H.gen(9700 + m)
    w = torch.randint(0, 256, (k, n // 2), generator=g, dtype=torch.uint8).numpy()
    ws = (torch.rand((k // 128, n), generator=g) * 0.02 + 0.002).to(torch.float16)
    x = torch.randn((m, k), generator=g).to(H.TORCH_DT[dtype])
    in_scale = np.array([0.03], np.float32)
    pqs = (in_scale[0] / (torch.rand(k, generator=g) * 1.5 + 0.5).numpy()).astype(np.float32)
    alpha = float(np.float32(0.03 * 0.8))
    w.tofile(tmp_path / "w.bin")
    H.bits_of(ws).tofile(tmp_path / "w_scale.bin")
    in_scale.tofile(tmp_path / "in_scale.bin")
    pqs.tofile(tmp_path / "pqs.bin")
    H.bits_of(x).tofile(tmp_path / "x.bin")
    run_driver("w4a8", tmp_path, TNAME[dtype], m, n, k, per_channel, repr(alpha))
    y = read_out(tmp_path / "y.bin", dtype, (m, n))
    xq = oracle.w4a8_static_quant(H.bits_of(x), pqs if per_channel else in_scale, bool(per_channel), dtype)
    ref = oracle.w4a8_gemm(xq, w.view(np.int8), H.bits_of(ws), alpha)
    H.check_gemm(y, ref, dtype, "w4a8 layer")


@pytest.mark.gpu
@pytest.mark.parametrize("m", [5, 200])
def test_w4a8_layer_group_64(tmp_path, oracle, m):
    """The layer with scale groups of 64 (the parameter struct's other group size)."""
    n, k, dtype = 512, 1024, H.BF16
    g = H.gen(9750 + m)
    w = torch.randint(0, 256, (k, n // 2), generator=g, dtype=torch.uint8).numpy()
    ws = (torch.rand((k // 64, n), generator=g) * 0.02 + 0.002).to(torch.float16)
    x = torch.randn((m, k), generator=g).to(H.TORCH_DT[dtype])
    in_scale = np.array([0.03], np.float32)
    alpha = float(np.float32(0.03 * 0.8))
    w.tofile(tmp_path / "w.bin")
    H.bits_of(ws).tofile(tmp_path / "w_scale.bin")
    in_scale.tofile(tmp_path / "in_scale.bin")
    H.bits_of(x).tofile(tmp_path / "x.bin")
    run_driver("w4a8", tmp_path, TNAME[dtype], m, n, k, 0, repr(alpha), 64)
    y = read_out(tmp_path / "y.bin", dtype, (m, n))
    xq = oracle.w4a8_static_quant(H.bits_of(x), in_scale, False, dtype)
    ref = oracle.w4a8_gemm(xq, w.view(np.int8), H.bits_of(ws), alpha, group=64)
    H.check_gemm(y, ref, dtype, "w4a8 layer, group 64")
