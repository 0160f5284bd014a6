"""Seeded random shapes of 33..512 rows in the three GEMM formats: the decode-form kernel over 32-row blocks and the MFMA
tile kernel (the library's small-problem rule on and off) must agree with each other and with a plain fp32 torch GEMM
on the dequantized operands - ragged last row blocks, column counts that are no multiple of 64 or 256, K from one
k-tile up.  The hand-picked cases of the other files are held against the CPU oracle; this file adds breadth."""
import random

import numpy as np
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu

REL = 5e-3


def _rel(a, b):
    a, b = a.float(), b.float()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def _shapes(seed, count):
    rng = random.Random(seed)
    return [(rng.randint(33, 512), 16 * rng.randint(1, 320), 128 * rng.randint(1, 40)) for _ in range(count)]


@pytest.mark.parametrize("M,N,K", _shapes(11, 16))
def test_w4a16_random_shapes(M, N, K):
    from ksanallm_amd import lib as L, ops
    rng = random.Random(M * 7 + N + K)
    dtype, awq = rng.choice([H.F16, H.BF16]), rng.random() < 0.5
    d = H.make_w4a16(9000 + M + N, M, N, K, 128, dtype, awq=awq, x_std=0.5, s_lo=0.002, s_hi=0.01, z_lo=0, z_hi=15)
    wp = ops.repack_weight(d["qweight"].cuda(), L.SRC_AWQ if awq else L.SRC_GPTQ, 1, K, N)
    sp = ops.repack_scales(d["scales"].cuda(), L.SCALE_GN, 1, K, N, 128)
    zp = ops.repack_zeros(d["qzeros"].cuda(), L.ZERO_AWQ_PACKED, K, N, 128) if awq else None
    out = {rule: ops.w4a16_gemm(d["x"].cuda(), wp, sp, zp, N, K, 128).clone() for rule in H.each_regime(M)}
    z = torch.from_numpy(d["zeros"].astype(np.float32)).cuda().repeat_interleave(128, 0) if awq else 8.0
    w = (torch.from_numpy(d["codes"].astype(np.float32)).cuda() - z) * d["scales"].cuda().float().repeat_interleave(128, 0)
    ref = d["x"].cuda().float() @ w
    assert _rel(out[True], ref) <= REL and _rel(out[False], ref) <= REL and _rel(out[True], out[False]) <= REL


@pytest.mark.parametrize("M,N,K", _shapes(12, 16))
def test_fp8_blockwise_random_shapes(M, N, K):
    from ksanallm_amd import ops
    g = H.gen(M + N + K)
    x = torch.randn((M, K), generator=g).to(torch.bfloat16).cuda()
    wq = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
    wq[(wq & 0x7F) == 0x7F] = 0x30  # no NaN encodings
    bs = torch.rand(((N + 127) // 128, K // 128), generator=g) * 1e-3 + 1e-4
    q, s = ops.per_token_group_quant_fp8(x, K, 128, True)
    bp = ops.fp8_repack_weight(wq.cuda())
    out = {rule: ops.fp8_blockwise_gemm(q, s, bp, bs.cuda(), torch.bfloat16).clone() for rule in H.each_regime(M)}
    wf = wq.cuda().view(torch.float8_e4m3fn).float() * bs.cuda().repeat_interleave(128, 0)[:N].repeat_interleave(128, 1)
    xf = q.view(torch.float8_e4m3fn).float() * s.t().contiguous().repeat_interleave(128, 1)
    ref = xf @ wf.t()
    assert _rel(out[True], ref) <= REL and _rel(out[False], ref) <= REL and _rel(out[True], out[False]) <= REL


@pytest.mark.parametrize("M,N,K", _shapes(13, 16))
def test_w4a8_random_shapes(oracle, M, N, K):
    from ksanallm_amd import ops
    g = H.gen(M + N + K)
    x = torch.randn((M, K), generator=g).to(torch.bfloat16).cuda()
    w = torch.randint(0, 256, (K, N // 2), generator=g, dtype=torch.uint8)
    scales = (torch.rand((K // 128, N), generator=g) * 0.02 + 0.002).to(torch.float16)
    xq, xsum = ops.w4a8_static_quant(x, torch.tensor([0.05], dtype=torch.float32).cuda(), False)
    wp = ops.w4a8_repack_weight(w.cuda())
    out = {rule: ops.w4a8_gemm(xq, xsum, wp, scales.cuda(), 0.03, N, torch.bfloat16).clone() for rule in H.each_regime(M)}
    assert _rel(out[True], out[False]) <= REL
    # the first 32 rows against the oracle (its int4 x e4m3 reference costs too much for all rows of every shape)
    ref = oracle.w4a8_gemm(xq[:32].cpu().numpy(), w.numpy().view(np.int8), H.bits_of(scales), 0.03)
    H.check_gemm(out[True][:32], ref, H.BF16, "w4a8 random M=%d N=%d K=%d" % (M, N, K))
