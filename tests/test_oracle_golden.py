"""Pins the CPU oracle against the known-answer vectors the reference's own tests hold (tests/golden/
reference_known_answers.json, each entry with the reference file:line it was taken from), and against what the
mathematics fixes.  No GPU."""
import json
import os

import numpy as np
import pytest
import torch

from tests import helpers as H

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")) as _f:
    GOLDEN = json.load(_f)


# ----------------------------------------------------------------------------- scalar formats
def test_f16_roundtrip_all_codes(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.f16_to_f32(bits)
    ref = torch.from_numpy(bits.view(np.int16)).view(torch.float16).float().numpy()
    ok = ~np.isnan(ref)  # NaN payloads may be quietened by the library
    np.testing.assert_array_equal(f.view(np.uint32)[ok], ref.view(np.uint32)[ok])
    assert np.all(np.isnan(f[~ok]))
    finite = np.isfinite(f)
    back = oracle.f32_to_f16(f[finite])
    np.testing.assert_array_equal(back, bits[finite])


def test_f32_to_f16_bf16_rne_matches_library(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10,
        (rng.standard_normal(50000) * 1e-6).astype(np.float32),
        np.float32([65504, 65519.99, 65520, 1e9, -1e9, 2.0**-24, 2.0**-25, 1.5 * 2.0**-24, 0.0, -0.0]),
    ])
    # ties: value exactly halfway between two halfs / bfloat16s
    ties = (np.arange(1, 4000, dtype=np.float32) * 2 + 1) * np.float32(2.0**-11)
    x = np.concatenate([x, ties, ties * 8])
    t = torch.from_numpy(x)
    np.testing.assert_array_equal(oracle.f32_to_f16(x), t.half().view(torch.int16).numpy().view(np.uint16))
    np.testing.assert_array_equal(oracle.f32_to_bf16(x), t.bfloat16().view(torch.int16).numpy().view(np.uint16))


def test_e4m3_decode_table(oracle):
    codes = np.arange(256, dtype=np.uint8)
    f = oracle.e4m3_to_f32(codes)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    ok = ~np.isnan(ref)
    np.testing.assert_array_equal(f[ok], ref[ok])
    assert np.isnan(f[0x7F]) and np.isnan(f[0xFF])
    assert f[0x7E] == 448.0 and f[0x01] == 2.0**-9 and f[0x08] == 2.0**-6


def test_e4m3_encode_rne_satfinite(oracle):
    # every code re-encodes to itself
    codes = np.array([c for c in range(256) if c & 0x7F != 0x7F], dtype=np.uint8)
    vals = oracle.e4m3_to_f32(codes)
    back = oracle.f32_to_e4m3(vals)
    # -0.0 keeps its sign bit
    np.testing.assert_array_equal(back, codes)
    # halfway points go to the even mantissa; values just off the tie go to the nearer neighbour
    pos = oracle.e4m3_to_f32(np.arange(0, 0x7F, dtype=np.uint8))
    mid = (pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2
    enc = oracle.f32_to_e4m3(mid.astype(np.float32))
    lo = np.arange(0, 0x7E, dtype=np.uint8)
    expect = np.where(lo % 2 == 0, lo, lo + 1)
    np.testing.assert_array_equal(enc, expect)
    np.testing.assert_array_equal(oracle.f32_to_e4m3(np.nextafter(mid.astype(np.float32), np.float32(0))), lo)
    np.testing.assert_array_equal(oracle.f32_to_e4m3(np.nextafter(mid.astype(np.float32), np.float32(1e9))), lo + 1)
    # round-to-nearest-even boundaries: 17->16, 19->20, 2^-10 -> 0, 1.5*2^-9 -> code 2
    got = oracle.e4m3_to_f32(oracle.f32_to_e4m3(np.float32([17, 19, 2.0**-10, 1.5 * 2.0**-9])))
    np.testing.assert_array_equal(got, np.float32([16, 20, 0, 2 * 2.0**-9]))
    # saturation instead of NaN, both signs; inf saturates, NaN stays NaN
    sat = oracle.f32_to_e4m3(np.float32([448, 449, 464, 465, 1e30, np.inf, -500, -np.inf]))
    np.testing.assert_array_equal(sat, np.uint8([0x7E] * 6 + [0xFE] * 2))
    assert oracle.f32_to_e4m3(np.float32([np.nan]))[0] & 0x7F == 0x7F
    # random cross-check against torch's cast inside the finite range
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(300000) * rng.choice([1e-3, 0.1, 1, 30, 200], 300000)).astype(np.float32)
    x = np.clip(x, -448, 448)
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(oracle.f32_to_e4m3(x), ref)


# ----------------------------------------------------------------------------- checkpoint layouts
def test_unpack_known_answer_0x66666666(oracle):
    """S/models/quant/cutlass_utils_test.cpp:80-108: int32 1717986918 everywhere -> every packed byte == -18."""
    fx = GOLDEN["unpack_0x66666666"]
    q = np.full(tuple(fx["shape"]), fx["input_word"], dtype=np.uint32)
    for unpack in (oracle.gptq_unpack, oracle.awq_unpack):
        codes = unpack(q)
        signed = (codes.astype(np.int16) - 8).astype(np.int8)
        packed = oracle.pack_int8_to_int4x2(signed)
        assert np.all(packed == fx["expected_packed_int8"])


def test_gptq_awq_unpack_positions(oracle):
    # one distinct nibble per position fixes the order
    word = sum(i << (4 * i) for i in range(8))  # nibble i holds value i
    g = oracle.gptq_unpack(np.full((1, 1), word, np.uint32))
    np.testing.assert_array_equal(g[:, 0], np.arange(8))
    a = oracle.awq_unpack(np.full((1, 1), word, np.uint32))
    # column 8j+i is read from nibble {0,4,1,5,2,6,3,7}[i]
    np.testing.assert_array_equal(a[0], [0, 4, 1, 5, 2, 6, 3, 7])
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 16, (64, 48), dtype=np.uint8)
    np.testing.assert_array_equal(oracle.gptq_unpack(oracle.gptq_pack(codes)), codes)
    np.testing.assert_array_equal(oracle.awq_unpack(oracle.awq_pack(codes)), codes)


def test_marlin_repack_golden(oracle):
    """S/models/quant/marlin_utils_test.cpp:29-91: arange(1024*1024) int32 viewed [1024,1024]."""
    t = np.arange(1024 * 1024, dtype=np.uint32).reshape(1024, 1024)
    awq = oracle.marlin_awq_repack(t)    # k=1024, n=8192
    gptq = oracle.marlin_gptq_repack(t)  # k=8192, n=1024
    fx = GOLDEN["marlin_repack_arange"]
    assert gptq.shape == tuple(fx["gptq_shape"]) and awq.shape == tuple(fx["awq_shape"])
    g, a = gptq.reshape(-1).view(np.int32), awq.reshape(-1).view(np.int32)
    np.testing.assert_array_equal(g[:10], fx["gptq_first10"])
    np.testing.assert_array_equal(a[:10], fx["awq_first10"])
    np.testing.assert_array_equal(g[-10:], fx["gptq_last10"])
    np.testing.assert_array_equal(a[-10:], fx["awq_last10"])


def test_marlin_awq_zero_points_golden(oracle):
    """S/models/quant/marlin_utils_test.cpp:149-173."""
    t = np.arange(1024 * 128, dtype=np.uint32).reshape(1024, 128)
    zp = oracle.marlin_awq_zero_points(t)
    fx = GOLDEN["marlin_awq_zero_points_arange"]
    assert zp.shape == tuple(fx["shape"])
    z = zp.reshape(-1).view(np.int32)
    np.testing.assert_array_equal(z[:10], fx["first10"])
    np.testing.assert_array_equal(z[-10:], fx["last10"])


def test_moe_layout_roundtrip_and_nibble_order(oracle):
    w = np.zeros((1, 2, 4), np.uint8)
    w[0, 1, 2] = 0xA3  # n=1, k=4 -> 3 ; k=5 -> 10
    codes = oracle.moe_unpack(w)
    assert codes[0, 4, 1] == 3 and codes[0, 5, 1] == 10 and codes.sum() == 13
    rng = np.random.default_rng(0)
    c = rng.integers(0, 16, (3, 32, 16), dtype=np.uint8)
    np.testing.assert_array_equal(oracle.moe_unpack(oracle.moe_pack(c)), c)


# ----------------------------------------------------------------------------- W4A16 numerics
def test_dequant_all_zero_codes_is_minus_8(oracle):
    """S/models/quant/quant_int4_weight_test.cpp:259-287 (CommonDeQuantTest)."""
    codes = np.zeros((256, 32), np.uint8)
    s = oracle.to_bits(np.ones((2, 32), np.float32), oracle.F16)
    w = oracle.w4a16_dequant(codes, s, None, 128, oracle.F16)
    assert np.all(w == GOLDEN["dequant_all_zero_codes"]["expected"])


@pytest.mark.parametrize("dtype", [0, 1])
def test_w4a16_gemm_vs_float64(oracle, dtype):
    rng = np.random.default_rng(3)
    M, N, K, G = 5, 96, 512, 128
    codes = rng.integers(0, 16, (K, N), dtype=np.uint8)
    zeros = rng.integers(6, 10, (K // G, N), dtype=np.uint8)
    s_bits = oracle.to_bits(rng.uniform(0.003, 0.015, (K // G, N)).astype(np.float32), dtype)
    x_bits = oracle.to_bits(rng.standard_normal((M, K)).astype(np.float32), dtype)
    s = oracle.from_bits(s_bits, dtype).astype(np.float64)
    x = oracle.from_bits(x_bits, dtype).astype(np.float64)
    for z in (None, zeros):
        zp = 8.0 if z is None else np.repeat(z, G, axis=0).astype(np.float64)
        wref = (codes.astype(np.float64) - zp) * np.repeat(s, G, axis=0)
        yref = x @ wref
        y = oracle.w4a16_gemm(x_bits, codes, s_bits, z, G, dtype)
        assert np.abs(y - yref).max() < 2e-5 * np.abs(yref).max() + 1e-5
        w = oracle.w4a16_dequant(codes, s_bits, z, G, dtype)
        np.testing.assert_array_equal(w, wref.astype(np.float32))
        y64 = oracle.gemm_xw_f64(x_bits, w, dtype)
        np.testing.assert_allclose(y64, yref, rtol=1e-12, atol=1e-12)


# ----------------------------------------------------------------------------- fp8 quantizer
TARGET_Q = GOLDEN["fp8_group_quant_i_over_100"]["codes"]


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("n", [128, 256])
@pytest.mark.parametrize("colmajor", [False, True])
def test_fp8_group_quant_known_answer(oracle, dtype, n, colmajor):
    """K/others/sglang/main/quantization/fp8/per_token_group_quant_test.cu:77-98: x[i] = i/100, m = 1;
    scales {0.0028, 0.0057} within 1e-4, codes within +-1 of the table (the table is shared by fp16 and bf16)."""
    x = (np.arange(n, dtype=np.float32) / np.float32(100.0)).reshape(1, n)
    xb = oracle.to_bits(x, dtype)
    q, s = oracle.fp8_group_quant(xb, n, 128, colmajor, False, dtype)
    s = s.reshape(-1)
    fx = GOLDEN["fp8_group_quant_i_over_100"]
    np.testing.assert_allclose(s, fx["scales"][: n // 128], atol=fx["scale_atol"])
    diff = np.abs(q.reshape(-1).astype(int) - np.array(TARGET_Q[:n]))
    assert diff.max() <= fx["code_tolerance"]
    assert (diff == 0).mean() > 0.95


def test_fp8_group_quant_closed_form(oracle):
    rng = np.random.default_rng(5)
    m, k = 7, 384
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[rng.random((m, k)) < 0.01] *= 20
    x[3, 128:256] = 0  # an all-zero group hits the 1e-10 floor
    for dtype in (0, 1):
        xb = oracle.to_bits(x, dtype)
        xr = oracle.from_bits(xb, dtype)
        q, s = oracle.fp8_group_quant(xb, k, 128, False, False, dtype)
        q2, s2 = oracle.fp8_group_quant(xb, k, 128, True, False, dtype)
        np.testing.assert_array_equal(q, q2)
        np.testing.assert_array_equal(s, s2.T)
        amax = np.maximum(np.abs(xr).reshape(m, 3, 128).max(-1), np.float32(1e-10))
        np.testing.assert_array_equal(s, amax / np.float32(448.0))
        assert s[3, 1] == np.float32(1e-10) / np.float32(448.0) and np.all(q[3, 128:256] == 0)
        # library cross-check: IEEE divide then torch's RNE cast (inputs never exceed 448 in magnitude)
        r = xr.reshape(m, 3, 128) / s[:, :, None]
        ref = torch.from_numpy(np.clip(r, -448, 448).reshape(m, k)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        np.testing.assert_array_equal(q, ref)
        # the group's largest element always lands on +-448
        assert np.all(np.abs(oracle.e4m3_to_f32(q)).reshape(m, 3, 128).max(-1)[amax > 1e-10] == 448.0)


def test_fp8_group_quant_fused_silu_close_to_unfused(oracle):
    rng = np.random.default_rng(6)
    m, k = 4, 256
    gu = rng.standard_normal((m, 2 * k)).astype(np.float32)
    for dtype in (0, 1):
        b = oracle.to_bits(gu, dtype)
        f = oracle.from_bits(b, dtype)
        act = oracle.to_bits(f[:, :k] / (1 + np.exp(-f[:, :k])) * f[:, k:], dtype)
        q0, s0 = oracle.fp8_group_quant(act, k, 128, True, False, dtype)
        q1, s1 = oracle.fp8_group_quant(b, k, 128, True, True, dtype)
        np.testing.assert_allclose(s1, s0, rtol=2e-2)
        assert (np.abs(q1.astype(int) - q0.astype(int)) <= 1).mean() > 0.99


# ----------------------------------------------------------------------------- blockwise fp8 GEMM
def test_fp8_blockwise_gemm_vs_float64(oracle):
    rng = np.random.default_rng(7)
    m, n, k = 5, 200, 384  # n not a multiple of 128: last scale row is partial
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    bq, bs = oracle.fp8_block_quant_weight(w)
    assert bs.shape == (2, 3)
    x = rng.standard_normal((m, k)).astype(np.float32)
    aq, a_s = oracle.fp8_group_quant(oracle.to_bits(x, 1), k, 128, True, False, 1)
    out = oracle.fp8_blockwise_gemm(aq, a_s, bq, bs, True)
    out_rm = oracle.fp8_blockwise_gemm(aq, np.ascontiguousarray(a_s.T), bq, bs, False)
    np.testing.assert_array_equal(out, out_rm)
    A = oracle.e4m3_to_f32(aq).astype(np.float64) * np.repeat(a_s.T.astype(np.float64), 128, axis=1)
    B = oracle.e4m3_to_f32(bq).astype(np.float64) * np.repeat(np.repeat(bs.astype(np.float64), 128, 0)[:n], 128, 1)
    ref = A @ B.T
    assert np.abs(out - ref).max() < 1e-5 * np.abs(ref).max()
    # quantization itself stays close to the unquantized product
    full = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.linalg.norm(ref - full) / np.linalg.norm(full) < 0.06
    # weight block scale = amax/448 and block maxima land on 448
    blk = np.abs(w[:128, :128]).max()
    assert bs[0, 0] == np.float32(blk) / np.float32(448.0)


# ----------------------------------------------------------------------------- MoE
def test_moe_align_worked_example(oracle):
    """K/moe_utils/moe_utils.cu:150-156."""
    fx = GOLDEN["moe_align_worked_example"]
    sorted_ids, expert_ids, npp = oracle.moe_align(fx["topk_ids"], fx["experts"], fx["block"])
    np.testing.assert_array_equal(sorted_ids[:20], fx["sorted_ids_first20"])   # 9 = the pad value numel
    assert npp == fx["num_tokens_post_pad"]
    np.testing.assert_array_equal(expert_ids[:5], fx["expert_ids_first5"])


def test_moe_align_invariants(oracle):
    rng = np.random.default_rng(8)
    for E, bm, numel in [(256, 16, 8), (256, 64, 4096), (8, 4, 0), (3, 1, 50)]:
        ids = rng.integers(0, E, numel).astype(np.int32)
        s, e, npp = oracle.moe_align(ids, E, bm)
        counts = np.bincount(ids, minlength=E)
        assert npp == int((np.ceil(counts / bm) * bm).sum())
        assert np.all(s[npp:] == numel)
        real = s[:npp][s[:npp] < numel]
        assert sorted(real.tolist()) == list(range(numel))
        for b in range(npp // bm):
            seg = s[b * bm:(b + 1) * bm]
            seg = seg[seg < numel]
            assert np.all(ids[seg] == e[b]) and np.all(np.diff(seg) > 0)
        # stable: inside an expert ids ascend across blocks too
        for ex in np.unique(ids):
            pos = real[ids[real] == ex]
            assert np.all(np.diff(pos) > 0)


def test_moe_gemm_matches_dense_dequant(oracle):
    rng = np.random.default_rng(9)
    E, N, K, G, T, topk = 6, 32, 256, 128, 5, 2
    codes = rng.integers(0, 16, (E, K, N), dtype=np.uint8)
    w = oracle.moe_pack(codes)
    dtype = 1
    s_bits = oracle.to_bits(rng.uniform(0.002, 0.01, (E, N, K // G)).astype(np.float32), dtype)
    x_bits = oracle.to_bits(rng.standard_normal((T, K)).astype(np.float32), dtype)
    ids = np.stack([rng.choice(E, topk, replace=False) for _ in range(T)]).astype(np.int32)
    tw = rng.random((T, topk)).astype(np.float32)
    out = oracle.moe_w4a16_gemm(x_bits, w, s_bits, ids, tw, topk, G, True, dtype)
    x = oracle.from_bits(x_bits, dtype).astype(np.float64)
    s = oracle.from_bits(s_bits, dtype).astype(np.float64)
    for t in range(T):
        for j in range(topk):
            e = ids[t, j]
            wd = (codes[e].astype(np.float64) - 8) * np.repeat(s[e].T, G, axis=0)  # [K, N]
            ref = x[t] @ wd * tw[t, j]
            np.testing.assert_allclose(out[t * topk + j], ref, rtol=1e-4, atol=1e-5)


def test_silu_mul_and_moe_sum(oracle):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    for dtype in (0, 1):
        xb = oracle.to_bits(x, dtype)
        xf = oracle.from_bits(xb, dtype)
        out = oracle.from_bits(oracle.silu_mul(xb, dtype), dtype)
        ref = oracle.from_bits(oracle.to_bits(xf[:, :32] / (1 + np.exp(-xf[:, :32])) * xf[:, 32:], dtype), dtype)
        assert np.abs(out - ref).max() <= np.abs(ref).max() * 2.0**-7
        y = rng.standard_normal((2, 8, 16)).astype(np.float32)
        yb = oracle.to_bits(y, dtype)
        tt = torch.from_numpy(oracle.from_bits(yb, dtype)).to(torch.float16 if dtype == 0 else torch.bfloat16)
        acc = torch.zeros_like(tt[:, 0])
        for j in range(8):
            acc = acc + tt[:, j]
        np.testing.assert_array_equal(oracle.from_bits(oracle.moe_sum(yb, dtype), dtype), acc.float().numpy())


def test_topk_softmax_vs_torch(oracle):
    g = torch.Generator().manual_seed(3)
    logits = torch.randn((37, 256), generator=g)
    w, ids = oracle.moe_topk_softmax(logits.numpy(), 8, False, 2.5, oracle.F32)
    p = torch.softmax(logits, -1)
    tw, ti = torch.topk(p, 8, dim=-1)
    np.testing.assert_array_equal(ids, ti.numpy())
    np.testing.assert_allclose(w, tw.numpy() * 2.5, rtol=1e-5)
    w2, _ = oracle.moe_topk_softmax(logits.numpy(), 8, True, 1.0, oracle.F32)
    np.testing.assert_allclose(w2.sum(-1), 1.0, rtol=1e-5)
    # ties go to the lower expert id
    flat = np.zeros((1, 16), np.float32)
    _, ids = oracle.moe_topk_softmax(flat, 4, False, 1.0, oracle.F32)
    np.testing.assert_array_equal(ids[0], [0, 1, 2, 3])


def _grouped_topk_torch(logits, bias, top_k, groups, topk_group, sigmoid, renorm, scaling):
    """The published DeepSeek-V2/V3 routing formula with tensor ops (the form S/kernels/nvidia/moe_kernel_wrapper.cpp:286-347
    spells out): an independent statement of what the oracle's loops compute."""
    T, E = logits.shape
    scores = torch.sigmoid(logits) if sigmoid else torch.softmax(logits, -1)
    original = scores
    if bias is not None:
        scores = scores + bias
        group_scores = scores.view(T, groups, -1).topk(2, -1)[0].sum(-1)
    else:
        group_scores = scores.view(T, groups, -1).max(-1)[0]
    group_idx = torch.topk(group_scores, topk_group, -1)[1]
    mask = torch.zeros_like(group_scores).scatter_(1, group_idx, 1)
    score_mask = mask.unsqueeze(-1).expand(T, groups, E // groups).reshape(T, -1)
    tmp = scores.masked_fill(~score_mask.bool(), float("-inf"))
    ids = torch.topk(tmp, top_k, -1)[1]
    w = original.gather(1, ids)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return w * scaling, ids


@pytest.mark.parametrize("E,top_k,groups,topk_group,sigmoid,use_bias,renorm", [
    (256, 8, 8, 4, True, True, True),      # DeepSeek-V3 (the reference test's first config)
    (128, 4, 4, 2, True, True, True),      # the reference test's second config
    (160, 6, 8, 3, False, False, False),   # DeepSeek-V2: softmax, group rank = max, no renormalisation
    (64, 6, 1, 1, True, False, True),      # ungrouped sigmoid
    (60, 4, 1, 1, False, False, True),     # ungrouped softmax, E not a multiple of 64
])
def test_grouped_topk_vs_torch(oracle, E, top_k, groups, topk_group, sigmoid, use_bias, renorm):
    g = torch.Generator().manual_seed(E + top_k)
    logits = torch.rand((301, E), generator=g) * 1.98 - 0.99      # U(-0.99, 0.99) as in the reference's test
    bias = (torch.rand(E, generator=g) * 0.009 - 0.01) if use_bias else None   # U(-0.01, -0.001)
    w, ids = oracle.moe_grouped_topk(logits.numpy(), None if bias is None else bias.numpy(), top_k, groups, topk_group,
                                     sigmoid, renorm, 2.5, oracle.F32)
    tw, ti = _grouped_topk_torch(logits, bias, top_k, groups, topk_group, sigmoid, renorm, 2.5)
    np.testing.assert_array_equal(ids, ti.numpy())
    np.testing.assert_allclose(w, tw.numpy(), rtol=2e-5)
    if renorm:
        np.testing.assert_allclose(w.sum(-1), 2.5, rtol=1e-5)   # the reference test's EXPECT_NEAR(sum, routed_scaling_factor)
    # every pick lies in a kept group: at most topk_group distinct groups per token
    per = E // groups
    assert max(len(set((row // per).tolist())) for row in ids) <= topk_group


# The reference's own host implementation of the router (compiled from the reference tree into oracle/_ref by
# `make -C oracle ref`; it exists for fp32 logits, sigmoid scoring with a correction bias and renormalized weights):
# same picks per token, same weight per pick.  Its heap returns a token's picks in another order, so picks are compared
# as sets and weights by expert id.
@pytest.mark.parametrize("T,E,top_k,groups,topk_group", [(301, 256, 8, 8, 4), (64, 128, 4, 4, 2), (17, 64, 6, 4, 3)])
def test_grouped_topk_vs_reference_host_code(oracle, T, E, top_k, groups, topk_group):
    g = torch.Generator().manual_seed(7 * E + T)
    logits = (torch.rand((T, E), generator=g) * 1.98 - 0.99).numpy()
    bias = (torch.rand(E, generator=g) * 0.009 - 0.01).numpy()
    ref = oracle.ref_grouped_topk(logits, bias, top_k, groups, topk_group, 2.5)
    if ref is None:
        pytest.skip("oracle/_ref is not built (the reference tree is not on this machine)")
    rw, ri = ref
    w, ids = oracle.moe_grouped_topk(logits, bias, top_k, groups, topk_group, True, True, 2.5, oracle.F32)
    for t in range(T):
        assert sorted(ids[t].tolist()) == sorted(ri[t].tolist()), t
        mine = dict(zip(ids[t].tolist(), w[t].tolist()))
        for e, x in zip(ri[t].tolist(), rw[t].tolist()):
            assert abs(mine[e] - x) <= 2e-6 * 2.5, (t, e, mine[e], x)


def test_grouped_topk_ties_and_group_rank(oracle):
    # 2 groups of 4; group 1 holds the single largest value but group 0 the larger top-2 sum: with a bias the rank is
    # the top-2 sum (group 0 kept), without it the maximum (group 1 kept)
    logits = np.array([[2.0, 2.0, -5, -5, 3.0, -5, -5, -5]], np.float32)
    zero = np.zeros(8, np.float32)
    _, ids = oracle.moe_grouped_topk(logits, zero, 2, 2, 1, True, True, 1.0, oracle.F32)
    np.testing.assert_array_equal(ids[0], [0, 1])      # equal scores: lower id first
    w, ids = oracle.moe_grouped_topk(logits, None, 2, 2, 1, True, False, 1.0, oracle.F32)
    np.testing.assert_array_equal(ids[0], [4, 5])
    np.testing.assert_allclose(w[0], [1 / (1 + np.exp(-3.0)), 1 / (1 + np.exp(5.0))], rtol=1e-6)
    # weights come from the unbiased score: a large bias changes the pick, not the weight
    bias = np.array([0, 0, 0, 10, 0, 0, 0, 0], np.float32)
    w, ids = oracle.moe_grouped_topk(logits, bias, 1, 1, 1, True, False, 1.0, oracle.F32)
    assert ids[0, 0] == 3
    np.testing.assert_allclose(w[0, 0], 1 / (1 + np.exp(5.0)), rtol=1e-6)


@pytest.mark.parametrize("channels,size", [(1, 31), (1, 5120), (3, 4096)])
def test_fp8_channel_quant_vs_torch_float8(oracle, channels, size):
    g = torch.Generator().manual_seed(size)
    x = (torch.randn((channels, size), generator=g) * 3).to(torch.bfloat16)
    x[0, 0] = 0.0
    q, s = oracle.fp8_channel_quant(H.bits_of(x), H.BF16)
    # the reference test's own formula for the scale (utils_test.cu:48-56)
    amax = x.float().abs().amax(-1).numpy()
    np.testing.assert_array_equal(s, np.maximum(amax / np.float32(448.0), np.float32(1.0 / 448.0 / 512.0)).astype(np.float32))
    # codes: torch's float8_e4m3fn conversion (round to nearest even) of the clamped quotient
    r = torch.clamp(x.float() / torch.from_numpy(s)[:, None], -448.0, 448.0)
    np.testing.assert_array_equal(q, r.to(torch.float8_e4m3fn).view(torch.uint8).numpy())
    # static: a given scale is used as is; an all-zero tensor takes the minimum scale
    q2, s2 = oracle.fp8_channel_quant(H.bits_of(x), H.BF16, scale=np.full(channels, 0.05, np.float32))
    r2 = torch.clamp(x.float() / 0.05, -448.0, 448.0)
    np.testing.assert_array_equal(q2, r2.to(torch.float8_e4m3fn).view(torch.uint8).numpy())
    _, s0 = oracle.fp8_channel_quant(np.zeros((1, 16), np.uint16), H.BF16)
    assert s0[0] == np.float32(1.0 / 448.0 / 512.0)


def test_fp8_tensor_gemm_vs_torch(oracle):
    g = torch.Generator().manual_seed(9)
    a = torch.randint(0, 256, (5, 256), generator=g, dtype=torch.uint8)
    b = torch.randint(0, 256, (7, 256), generator=g, dtype=torch.uint8)
    a = torch.where((a & 0x7f) == 0x7f, a & 0xfe, a)
    b = torch.where((b & 0x7f) == 0x7f, b & 0xfe, b)
    out = oracle.fp8_tensor_gemm(a.numpy(), 0.01, b.numpy(), 0.002)
    ref = (a.view(torch.float8_e4m3fn).double() @ b.view(torch.float8_e4m3fn).double().T) * np.float32(0.01) * np.float32(0.002)
    np.testing.assert_allclose(out, ref.numpy(), rtol=1e-6)


def test_act_order_definition(oracle):
    g = torch.Generator().manual_seed(11)
    K, N, M, group = 256, 32, 3, 128
    codes = torch.randint(0, 16, (K, N), generator=g, dtype=torch.uint8).numpy()
    scales = H.uniform(g, (K // group, N), 0.004, 0.02, H.F16)
    x = torch.randn((M, K), generator=g).to(torch.float16)
    # without act-order (g_idx = k // group) the definition is the plain group-wise GEMM
    plain = oracle.w4a16_gemm(H.bits_of(x), codes, H.bits_of(scales), None, group, H.F16)
    same = oracle.gptq_act_order_gemm(H.bits_of(x), codes, H.bits_of(scales), np.arange(K) // group, H.F16)
    np.testing.assert_allclose(same, plain, rtol=2e-5, atol=2e-5)
    # with a shuffled g_idx: brute force, element by element
    g_idx = (torch.randperm(K, generator=g) // group).numpy()
    y = oracle.gptq_act_order_gemm(H.bits_of(x), codes, H.bits_of(scales), g_idx, H.F16)
    xs, ss = x.double().numpy(), scales.double().numpy()
    brute = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            brute[m, n] = sum(xs[m, k] * (float(codes[k, n]) - 8.0) * ss[g_idx[k], n] for k in range(K))
    np.testing.assert_allclose(y, brute, rtol=1e-6, atol=1e-6)
    # sorting the rows by g_idx and permuting x the same way (what the GPU path does) gives the same product
    perm = np.argsort(g_idx, kind="stable")
    assert np.array_equal(g_idx[perm], np.arange(K) // group)
    moved = oracle.w4a16_gemm(H.bits_of(x[:, torch.from_numpy(perm)].contiguous()), codes[perm], H.bits_of(scales), None, group, H.F16)
    np.testing.assert_allclose(moved, y, rtol=2e-5, atol=2e-5)


def test_fp8_weight_fragment_layout_by_definition(oracle):
    """The packed fp8 layout, element by element from its definition: fragment (e, n/16, k/128) of 2 KiB; inside, half h,
    lane l = 16*((k%128)/32) + n%16, byte k%16 - against the oracle's vectorised permutation."""
    g = torch.Generator().manual_seed(21)
    E, N, K = 2, 32, 256
    w = torch.randint(0, 256, (E, N, K), generator=g, dtype=torch.uint8).numpy()
    p = oracle.fp8_repack_weight(w).reshape(-1)
    KB = K // 128
    for e in range(E):
        for n in range(N):
            for k in range(K):
                frag = (e * (N // 16) + n // 16) * KB + k // 128
                h = (k % 32) // 16
                lane = 16 * ((k % 128) // 32) + n % 16
                assert p[frag * 2048 + h * 1024 + lane * 16 + k % 16] == w[e, n, k]
    # 2-D input is the E = 1 case
    np.testing.assert_array_equal(oracle.fp8_repack_weight(w[0]), oracle.fp8_repack_weight(w[:1])[0])


def test_moe_act_order_forward_reduces_to_the_plain_block(oracle):
    """The act-order MoE oracle (scale[g_idx[k]] per weight row, by definition) against the pinned plain block:
      * with g_idx[k] = k // 128 the two are the same function;
      * with a shuffled g_idx it equals the plain block run on experts whose rows are sorted by group and on activations
        whose columns are permuted the same way - the route the reference takes (marlin_moe_layer.cpp:71-93)."""
    rng = np.random.default_rng(21)
    E, hidden, inter, topk, T = 4, 256, 128, 2, 5
    dtype = 0

    def experts(n, k):
        codes = rng.integers(0, 16, (E, k, n), dtype=np.uint8)               # [E, k, n], checkpoint row order
        scales = oracle.to_bits((rng.random((E, k // 128, n)) * 0.01 + 0.002).astype(np.float32), dtype)
        return codes, scales

    def as_moe_bytes(codes, scales_bits):                                      # [E, n, k/2] bytes, [E, n, k/128] scales
        c = codes.transpose(0, 2, 1)
        return (c[:, :, 0::2] | (c[:, :, 1::2] << 4)).astype(np.uint8), np.ascontiguousarray(scales_bits.transpose(0, 2, 1))

    c13, s13 = experts(2 * inter, hidden)
    c2, s2 = experts(hidden, inter)
    x = oracle.to_bits(rng.standard_normal((T, hidden)).astype(np.float32), dtype)
    ids = np.stack([rng.choice(E, topk, replace=False) for _ in range(T)]).astype(np.int32)
    tw = rng.random((T, topk)).astype(np.float32)
    nat13 = np.tile(np.arange(hidden) // 128, (E, 1)).astype(np.int32)
    nat2 = np.tile(np.arange(inter) // 128, (E, 1)).astype(np.int32)
    w13b, s13b = as_moe_bytes(c13, s13)
    w2b, s2b = as_moe_bytes(c2, s2)
    plain = oracle.moe_forward(x, w13b, s13b, w2b, s2b, ids, tw, 128, dtype)
    np.testing.assert_array_equal(oracle.moe_act_order_forward(x, c13, s13, nat13, c2, s2, nat2, ids, tw, dtype), plain)

    # shuffled groups on the first GEMM only (the second keeps natural order so that one permutation is in play):
    # one expert per token, so that a single column permutation of x describes the reference's route
    g13 = np.stack([rng.permutation(hidden) // 128 for _ in range(E)]).astype(np.int32)
    ids1 = ids[:, :1].copy()
    tw1 = tw[:, :1].copy()
    got = oracle.moe_act_order_forward(x, c13, s13, g13, c2, s2, nat2, ids1, tw1, dtype)
    for t in range(T):
        e = int(ids1[t, 0])
        perm = np.argsort(g13[e], kind="stable")
        c13s = c13.copy()
        c13s[e] = c13[e][perm]
        w13s, _ = as_moe_bytes(c13s, s13)
        xt = np.ascontiguousarray(x[t:t + 1][:, perm])
        ref = oracle.moe_forward(xt, w13s, s13b, w2b, s2b, ids1[t:t + 1], tw1[t:t + 1], 128, dtype)
        # same products in another order inside each group sum: equal up to one rounding of the 16-bit results
        a = oracle.from_bits(got[t:t + 1], dtype).astype(np.float64)
        b = oracle.from_bits(ref, dtype).astype(np.float64)
        assert np.max(np.abs(a - b)) <= 2e-3 * max(1.0, np.max(np.abs(b)))
