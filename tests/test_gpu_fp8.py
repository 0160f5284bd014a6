"""FP8 per-token-group quantizer (bit-exact codes and scales) and the blockwise FP8 GEMM."""
import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.test_oracle_golden import TARGET_Q

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from ksanallm_amd import ops
    return ops


def make_act(seed, m, k, dtype):
    g = H.gen(seed)
    x = torch.randn((m, k), generator=g)
    mask = torch.rand((m, k), generator=g) < 0.01
    x = torch.where(mask, x * 20, x)
    return x.to(H.TORCH_DT[dtype])


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("n", [128, 256])
@pytest.mark.parametrize("colmajor", [False, True])
def test_quant_known_answer(ops, oracle, dtype, n, colmajor):
    """Reference vector: x[i] = i/100 (per_token_group_quant_test.cu:77-98)."""
    x = (torch.arange(n, dtype=torch.float32) / 100.0).to(H.TORCH_DT[dtype]).view(1, n)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), n, 128, colmajor)
    qo, so = oracle.fp8_group_quant(H.bits_of(x), n, 128, colmajor, False, dtype)
    np.testing.assert_array_equal(q.cpu().numpy(), qo)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))
    assert np.abs(q.cpu().numpy().reshape(-1).astype(int) - np.array(TARGET_Q[:n])).max() <= 1
    np.testing.assert_allclose(s.cpu().numpy().reshape(-1), [0.0028, 0.0057][: n // 128], atol=1e-4)


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("m,k,group", [(1, 7168, 128), (16, 18432, 128), (37, 1024, 64), (5, 256, 32), (128, 7168, 128)])
@pytest.mark.parametrize("colmajor", [False, True])
def test_quant_bit_exact(ops, oracle, dtype, m, k, group, colmajor):
    x = make_act(4000 + m + k, m, k, dtype)
    if m > 2:
        x[1, :group] = 0          # all-zero group: scale floor 1e-10/448
        x[2, :group] *= 1e-4      # tiny values: subnormal codes
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, group, colmajor)
    qo, so = oracle.fp8_group_quant(H.bits_of(x), k, group, colmajor, False, dtype)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))
    np.testing.assert_array_equal(q.cpu().numpy(), qo)


@pytest.mark.parametrize("m,k,group", [(1, 7168, 128), (37, 1024, 64), (5, 256, 32), (130, 2048, 128)])
@pytest.mark.parametrize("colmajor", [False, True])
def test_quant_fp32_activations_bit_exact(ops, oracle, m, k, group, colmajor):
    """The float instantiation of the reference's quantizer: 24-bit mantissas in, IEEE divisions throughout."""
    g = H.gen(4040 + m + k)
    x = torch.randn((m, k), generator=g)
    x = torch.where(torch.rand((m, k), generator=g) < 0.01, x * 20, x)
    if m > 2:
        x[1, :group] = 0          # all-zero group: scale floor 1e-10/448
        x[2, :group] *= 1e-30     # values far below the floor's scale: codes of zero
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, group, colmajor)
    qo, so = oracle.fp8_group_quant(x.numpy(), k, group, colmajor, False, oracle.F32)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))
    np.testing.assert_array_equal(q.cpu().numpy(), qo)


def test_blockwise_gemm_fp32_activations(ops, oracle):
    """fp32 in, fp32 out (InvokeBlockGemm<float>): the quantizer's float form in front of the GEMM whose sums are the
    output, in both kernel regimes."""
    for (m, n, k) in [(7, 512, 1024), (130, 2304, 1152)]:
        g = H.gen(4060 + m)
        w = (torch.randn((n, k), generator=g) * 0.02).to(torch.bfloat16).float().numpy()
        bq, bs = oracle.fp8_block_quant_weight(w)
        x = torch.randn((m, k), generator=g)
        q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
        qo, so = oracle.fp8_group_quant(x.numpy(), k, 128, True, False, oracle.F32)
        np.testing.assert_array_equal(q.cpu().numpy(), qo)
        ref = oracle.fp8_blockwise_gemm(qo, so, bq, bs, True)
        for rule in H.each_regime(m):
            out = ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.float32)
            assert out.dtype == torch.float32
            H.check_gemm_f32(out, ref, "fp8 fp32 activations m=%d n=%d k=%d" % (m, n, k))


def test_quant_every_e4m3_boundary(ops, oracle):
    """Rows whose amax is exactly 448 make the scale 1, so the codes are the bare float->e4m3 conversion: sweep
    every representable value, every rounding midpoint and their neighbours."""
    pos = oracle.e4m3_to_f32(np.arange(0, 0x7F, dtype=np.uint8)).astype(np.float64)
    mid = (pos[:-1] + pos[1:]) / 2
    vals = np.concatenate([pos, mid]).astype(np.float32)
    vals = np.concatenate([vals, np.nextafter(vals, np.float32(0)), np.nextafter(vals, np.float32(1e9))])
    vals = vals[vals <= 448]
    vals = np.concatenate([vals, -vals])
    # fp16 cannot hold all of these; send them through a bf16/fp16-exact subset check instead: use fp16 where exact
    for dtype in (H.F16, H.BF16):
        v = torch.from_numpy(vals).to(H.TORCH_DT[dtype])
        n = v.numel()
        rows = (n + 126) // 127
        x = torch.zeros((rows, 128), dtype=v.dtype)
        x[:, 0] = 448.0
        flat = x[:, 1:].reshape(-1)
        flat[:n] = v
        x[:, 1:] = flat.view(rows, 127)
        q, s = ops.per_token_group_quant_fp8(x.cuda(), 128, 128, False)
        assert torch.all(s == 1.0)
        qo, _ = oracle.fp8_group_quant(H.bits_of(x), 128, 128, False, False, dtype)
        np.testing.assert_array_equal(q.cpu().numpy(), qo)


def test_quant_full_size_properties(ops, oracle):
    """M=4096, K=7168: every group's largest element encodes to +-448, dequantized values stay within half an e4m3
    step of the input, and a bounded sample of rows is bit-exact against the oracle."""
    m, k = 4096, 7168
    x = make_act(4444, m, k, H.BF16)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    lut = torch.from_numpy(oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8))).cuda()
    deq = lut[q.long()].view(m, k // 128, 128)
    assert torch.all(deq.abs().amax(-1) == 448.0)
    rec = deq * s.t().contiguous().view(m, k // 128, 1)
    err = (rec - x.cuda().float().view(m, k // 128, 128)).abs()
    assert torch.all(err <= s.t().contiguous().view(m, k // 128, 1) * 16.001 + 1e-12)  # half of the largest step (32), plus fp32 rounding of x/s
    rows = [0, 1, 777, 4095]
    qo, so = oracle.fp8_group_quant(H.bits_of(x[rows]), k, 128, True, False, H.BF16)
    np.testing.assert_array_equal(q[rows].cpu().numpy(), qo)
    np.testing.assert_array_equal(s[:, rows].cpu().numpy(), so)


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
def test_quant_fused_silu_mul(ops, oracle, dtype):
    """Tolerance check only: the reference's fused variant uses NVIDIA tanh.approx and is not pinned bit-exactly."""
    m, k = 9, 512
    g = H.gen(12)
    gu = torch.randn((m, 2 * k), generator=g).to(H.TORCH_DT[dtype])
    q, s = ops.per_token_group_quant_fp8(gu.cuda(), k, 128, True, fuse_silu_mul=True)
    qo, so = oracle.fp8_group_quant(H.bits_of(gu), k, 128, True, True, dtype)
    np.testing.assert_allclose(s.cpu().numpy(), so, rtol=2e-2)
    lut = oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8))
    a = lut[q.cpu().numpy()] * np.repeat(s.cpu().numpy().T, 128, axis=1)
    b = lut[qo] * np.repeat(so.T, 128, axis=1)
    assert np.linalg.norm(a - b) / np.linalg.norm(b) < 2e-2


def packed(ops, bq):
    """checkpoint-layout e4m3 weight (numpy) -> device tensor in the packed fragment layout the GEMMs read"""
    return ops.fp8_repack_weight(torch.from_numpy(bq).cuda())


def make_fp8_problem(oracle, seed, m, n, k, dtype=H.BF16):
    g = H.gen(seed)
    w = (torch.randn((n, k), generator=g) * 0.02).to(torch.bfloat16).float().numpy()
    bq, bs = oracle.fp8_block_quant_weight(w)
    x = make_act(seed + 1, m, k, dtype)
    return x, bq, bs


@pytest.mark.parametrize("m", [1, 16, 33, 128])
@pytest.mark.parametrize("n,k", [(512, 1024), (2304, 7168)])
def test_blockwise_gemm(ops, oracle, m, n, k):
    x, bq, bs = make_fp8_problem(oracle, 4100 + m + n, m, n, k)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    out = ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.bfloat16)
    # the oracle consumes the very codes and scales the GPU quantizer produced
    ref = oracle.fp8_blockwise_gemm(q.cpu().numpy(), s.cpu().numpy(), bq, bs, True)
    H.check_gemm(out, ref, H.BF16, "fp8 m=%d n=%d k=%d" % (m, n, k))


# the two shapes of the DeepSeek-V3 dense MLP benchmark at its decode and small-prefill row counts, against the oracle
@pytest.mark.parametrize("m", [1, 16, 128])
@pytest.mark.parametrize("n,k", [(18432, 7168), (7168, 18432)])
def test_blockwise_gemm_benchmark_shapes(ops, oracle, m, n, k):
    x, bq, bs = make_fp8_problem(oracle, 4150 + m + n, m, n, k)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    out = ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.bfloat16)
    ref = oracle.fp8_blockwise_gemm(q.cpu().numpy(), s.cpu().numpy(), bq, bs, True)
    H.check_gemm(out, ref, H.BF16, "fp8 cfg4 m=%d n=%d k=%d" % (m, n, k))


# the same two shapes at the benchmark's prefill row counts: the GPU multiplies all rows, the oracle the first 128 of
# them (rows are independent in the quantizer and in the GEMM), from the very codes and scales the GPU produced
@pytest.mark.parametrize("m", [1024, 4096])
@pytest.mark.parametrize("n,k", [(18432, 7168), (7168, 18432)])
def test_blockwise_gemm_benchmark_shapes_prefill_rows(ops, oracle, m, n, k):
    rows = 128
    x, bq, bs = make_fp8_problem(oracle, 4170 + m + n, m, n, k)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    qo, so = oracle.fp8_group_quant(H.bits_of(x[:rows]), k, 128, True, False, H.BF16)
    np.testing.assert_array_equal(q[:rows].cpu().numpy(), qo)
    np.testing.assert_array_equal(s[:, :rows].cpu().numpy().view(np.uint32), so.view(np.uint32))
    out = ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.bfloat16)
    ref = oracle.fp8_blockwise_gemm(qo, so, bq, bs, True)
    H.check_gemm(out[:rows], ref, H.BF16, "fp8 cfg4 m=%d n=%d k=%d, rows 0..%d" % (m, n, k, rows - 1))
    # and the last rows, which the last row tile and (at n = 7168) the cut tiles of the tail hold
    qo, so = oracle.fp8_group_quant(H.bits_of(x[m - 32:]), k, 128, True, False, H.BF16)
    ref = oracle.fp8_blockwise_gemm(qo, so, bq, bs, True)
    H.check_gemm(out[m - 32:], ref, H.BF16, "fp8 cfg4 m=%d n=%d k=%d, last 32 rows" % (m, n, k))


# prefill regime (MFMA tile kernel, 256 x 256 or 128 x 256 tiles): ragged M and N, odd k-block counts, split-K through
# the workspace
# (the last three: more than 32 tiles of 256 tokens, which is where the planner keeps that tile at these sizes)
@pytest.mark.parametrize("m,n,k,bm", [(65, 256, 128, 128), (300, 2320, 1152, 128), (256, 7168, 2048, 128), (1024, 512, 4096, 128),
                                      (130, 4096, 7168, 128), (128, 7168, 2048, 128), (384, 528, 1024, 128), (100, 272, 384, 128),
                                      (500, 768, 640, 128), (512, 4352, 256, 256), (200, 8704, 256, 256),
                                      (1024, 2304, 384, 256)])
def test_blockwise_gemm_tile_kernel(ops, oracle, m, n, k, bm, tile_kernels):
    from ksanallm_amd import lib as L
    desc = L.select_tile(L.KIND_FP8_BLOCKWISE, m, n, k, H.BF16)
    assert desc["kernel"] == 1 and desc["block_m"] == bm
    x, bq, bs = make_fp8_problem(oracle, 4400 + m + n, m, n, k)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    out = ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.bfloat16)
    ref = oracle.fp8_blockwise_gemm(q.cpu().numpy(), s.cpu().numpy(), bq, bs, True)
    H.check_gemm(out, ref, H.BF16, "fp8 tile m=%d n=%d k=%d split=%d" % (m, n, k, desc["split_k"]))
    if desc["split_k"] > 1:
        small = torch.empty(64, dtype=torch.uint8, device="cuda")
        with pytest.raises(L.KsqError) as e:
            ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.bfloat16,
                                   workspace=small)
        assert e.value.code == 3


# small problems of more than 32 tokens (ceil(m / 32) * n * k <= 5 * 2^24, m <= 512): the streaming kernel over blocks of
# 32 tokens, ragged last block included
@pytest.mark.parametrize("m,n,k", [(65, 256, 128), (100, 272, 384), (128, 4096, 4096), (300, 2320, 1152), (500, 768, 640),
                                   (33, 7168, 2048)])
def test_blockwise_gemm_row_blocks_above_32_tokens(ops, oracle, m, n, k):
    from ksanallm_amd import lib as L
    desc = L.select_tile(L.KIND_FP8_BLOCKWISE, m, n, k, H.BF16)
    assert desc["kernel"] == 0
    x, bq, bs = make_fp8_problem(oracle, 4450 + m + n, m, n, k)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    out = ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.bfloat16)
    ref = oracle.fp8_blockwise_gemm(q.cpu().numpy(), s.cpu().numpy(), bq, bs, True)
    H.check_gemm(out, ref, H.BF16, "fp8 row blocks m=%d n=%d k=%d" % (m, n, k))


# a little more than one round of tiles: the first 256 tiles are computed whole, the rest cut along K
def test_blockwise_gemm_whole_and_cut_tiles(ops, oracle, tile_kernels):
    from ksanallm_amd import lib as L
    m, n, k = 1030, 13328, 4096
    desc = L.select_tile(L.KIND_FP8_BLOCKWISE, m, n, k, H.BF16)
    tiles = 5 * 53
    assert desc["kernel"] == 1 and desc["split_k"] > 1 and desc["grid"] == 256 + (tiles - 256) * desc["split_k"]
    x, bq, bs = make_fp8_problem(oracle, 4500, m, n, k)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    out = ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.bfloat16)
    ref = oracle.fp8_blockwise_gemm(q.cpu().numpy(), s.cpu().numpy(), bq, bs, True)
    H.check_gemm(out, ref, H.BF16, "fp8 whole + cut tiles")


def test_blockwise_gemm_partial_scale_row_and_fp16_out(ops, oracle):
    m, n, k = 7, 208, 384  # n not a multiple of 128: the last scale row covers 80 weight rows
    x, bq, bs = make_fp8_problem(oracle, 4321, m, n, k, H.F16)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    out = ops.fp8_blockwise_gemm(q, s, packed(ops, bq), torch.from_numpy(bs).cuda(), torch.float16)
    ref = oracle.fp8_blockwise_gemm(q.cpu().numpy(), s.cpu().numpy(), bq, bs, True)
    H.check_gemm(out, ref, H.F16, "fp8 partial")


# ---- per-tensor / per-channel fp8 ------------------------------------------------------------------------------------

# the reference test's shapes (3rdparty/LLM_kernels/csrc/utils/nvidia/utils_test.cu:107) plus ragged / unaligned ones
@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("channels,size", [(1, 31), (1, 16383), (1, 5120), (1, 12800), (1, 4096), (64, 5120), (3, 77),
                                           (1, 4096 * 7168)])
def test_channel_quant_bit_exact(ops, oracle, dtype, channels, size):
    g = H.gen(channels + size)
    x = (torch.randn((channels, size), generator=g) * 2.5).to(H.TORCH_DT[dtype])
    q, s = ops.fp8_e4m3_quantize(x.cuda())
    qo, so = oracle.fp8_channel_quant(H.bits_of(x), dtype)
    np.testing.assert_array_equal(s.cpu().numpy(), so)
    np.testing.assert_array_equal(q.cpu().numpy(), qo)
    # static: given scales (values far outside the range saturate at +-448)
    given = torch.full((channels,), 0.004, dtype=torch.float32)
    q2, _ = ops.fp8_e4m3_quantize(x.cuda(), given.cuda())
    qo2, _ = oracle.fp8_channel_quant(H.bits_of(x), dtype, scale=given.numpy())
    np.testing.assert_array_equal(q2.cpu().numpy(), qo2)


@pytest.mark.parametrize("channels,size", [(1, 31), (1, 16383), (1, 5120), (64, 5120), (3, 77)])
def test_channel_quant_fp32_activations_bit_exact(ops, oracle, channels, size):
    """The float instantiation (Fp8E4m3Quantize<float>): 24-bit mantissas, IEEE divisions throughout."""
    g = H.gen(70 + channels + size)
    x = torch.randn((channels, size), generator=g) * 2.5
    q, s = ops.fp8_e4m3_quantize(x.cuda())
    qo, so = oracle.fp8_channel_quant(x.numpy(), oracle.F32)
    np.testing.assert_array_equal(s.cpu().numpy(), so)
    np.testing.assert_array_equal(q.cpu().numpy(), qo)
    given = torch.full((channels,), 0.004, dtype=torch.float32)
    q2, _ = ops.fp8_e4m3_quantize(x.cuda(), given.cuda())
    qo2, _ = oracle.fp8_channel_quant(x.numpy(), oracle.F32, scale=given.numpy())
    np.testing.assert_array_equal(q2.cpu().numpy(), qo2)


def test_channel_quant_zero_tensor_takes_minimum_scale(ops):
    x = torch.zeros((2, 64), dtype=torch.bfloat16, device="cuda")
    q, s = ops.fp8_e4m3_quantize(x)
    assert torch.all(s == 1.0 / 448.0 / 512.0) and torch.all(q == 0)


@pytest.mark.parametrize("m,n,k", [(1, 512, 1024), (16, 2304, 7168), (130, 4096, 1024), (1030, 13328, 512)])
def test_fp8_quantized_matmul(ops, oracle, m, n, k):
    g = H.gen(5100 + m + n)
    w = (torch.randn((n, k), generator=g) * 0.02).to(torch.bfloat16)
    x = make_act(5200 + m, m, k, H.BF16)
    wq, ws = ops.fp8_e4m3_quantize(w.reshape(1, -1).cuda())
    xq, xs = ops.fp8_e4m3_quantize(x.reshape(1, -1).cuda())
    wp = ops.fp8_repack_weight(wq.view(n, k))
    out = ops.fp8_quantized_matmul(xq.view(m, k), xs, wp, ws, torch.bfloat16)
    ref = oracle.fp8_tensor_gemm(xq.view(m, k).cpu().numpy(), xs.item(), wq.view(n, k).cpu().numpy(), ws.item())
    H.check_gemm(out, ref, H.BF16, "fp8 per-tensor m=%d n=%d k=%d" % (m, n, k))
    small = torch.empty(256, dtype=torch.uint8, device="cuda")
    from ksanallm_amd import lib as L
    with pytest.raises(L.KsqError) as e:
        ops.fp8_quantized_matmul(xq.view(m, k), xs, wp, ws, torch.bfloat16, workspace=small)
    assert e.value.code == 3


# ---- packed fragment layout of fp8 weights ---------------------------------------------------------------------------

@pytest.mark.parametrize("shape", [(16, 128), (48, 384), (3, 32, 256), (2320, 1152)])
def test_fp8_weight_repack_bit_exact_and_round_trip(ops, oracle, shape):
    g = H.gen(sum(shape))
    w = torch.randint(0, 256, shape, generator=g, dtype=torch.uint8)
    p = ops.fp8_repack_weight(w.cuda())
    np.testing.assert_array_equal(p.cpu().numpy(), oracle.fp8_repack_weight(w.numpy()))
    assert torch.equal(ops.fp8_unpack_weight(p).cpu(), w)


def test_fp8_weight_repack_rejects_bad_shapes(ops):
    from ksanallm_amd import lib as L
    for shape in ((8, 128), (16, 100)):
        with pytest.raises(L.KsqError) as e:
            ops.fp8_repack_weight(torch.zeros(shape, dtype=torch.uint8, device="cuda"))
        assert e.value.code == 1


@pytest.mark.parametrize("n,k", [(7168, 18432), (18432, 7168)])
def test_blockwise_gemm_full_size_properties(ops, oracle, n, k):
    """Size-independent properties of the fp8 tile kernel at the full benchmark shapes (M = 4096):
    doubling the activations doubles the scales and leaves the codes alone, so every output doubles exactly; permuting
    the rows of x permutes the rows of the output bit for bit."""
    m = 4096
    g = H.gen(4700 + n)
    b = torch.randint(0, 256, (n, k), generator=g, dtype=torch.uint8)
    b = torch.where((b & 0x7f) == 0x7f, b & 0xfe, b)          # no NaN codes
    bs = (torch.rand((n // 128, k // 128), generator=g) * 1e-4 + 1e-4).cuda()
    bp = ops.fp8_repack_weight(b.cuda())
    x = torch.randn((m, k), generator=g).to(torch.bfloat16).cuda()
    q, s = ops.per_token_group_quant_fp8(x, k, 128, True)
    y = ops.fp8_blockwise_gemm(q, s, bp, bs, torch.bfloat16)
    assert torch.all(torch.isfinite(y)) and y.abs().max() > 0
    q2, s2 = ops.per_token_group_quant_fp8(x * 2, k, 128, True)
    assert torch.equal(q2, q) and torch.equal(s2, s * 2)
    assert torch.equal(ops.fp8_blockwise_gemm(q2, s2, bp, bs, torch.bfloat16), y * 2)
    perm = torch.randperm(m, generator=g).cuda()
    qp, sp = ops.per_token_group_quant_fp8(x[perm].contiguous(), k, 128, True)
    assert torch.equal(ops.fp8_blockwise_gemm(qp, sp, bp, bs, torch.bfloat16), y[perm])


# the sums before they are rounded to bf16 (ksq_fp8_blockwise_gemm_f32: same kernels, same plan): the parity bar as
# written, raw - streaming kernel, tile kernel with whole tiles, tile kernel with tiles cut along K
@pytest.mark.parametrize("m,n,k", [(1, 18432, 7168), (16, 7168, 18432), (128, 7168, 18432), (128, 18432, 7168),
                                   (300, 2320, 1152), (1024, 2304, 384)])
def test_blockwise_gemm_sums_before_output_rounding(ops, oracle, m, n, k):
    x, bq, bs = make_fp8_problem(oracle, 4800 + m + n, m, n, k)
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, True)
    bp, bsd = packed(ops, bq), torch.from_numpy(bs).cuda()
    ref = oracle.fp8_blockwise_gemm(q.cpu().numpy(), s.cpu().numpy(), bq, bs, True)
    for rule in H.each_regime(m):
        y32 = ops.fp8_blockwise_gemm_f32(q, s, bp, bsd)
        y = ops.fp8_blockwise_gemm(q, s, bp, bsd, torch.bfloat16)
        assert torch.equal(y32.to(torch.bfloat16).view(torch.int16), y.view(torch.int16))
        H.check_gemm_f32(y32, ref, "fp8 before rounding m=%d n=%d k=%d, small-problem rule %s" % (m, n, k, rule))