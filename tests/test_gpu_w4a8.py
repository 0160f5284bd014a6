"""W4A8: weight repack (bit-exact), static e4m3 quantizer with group sums (bit-exact), GEMM (GEMM tolerance)."""
import numpy as np
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from ksanallm_amd import ops
    return ops


def make_weight(seed, k, n):
    g = H.gen(seed)
    w = torch.randint(0, 256, (k, n // 2), generator=g, dtype=torch.uint8)
    scales = (torch.rand((k // 128, n), generator=g) * 0.02 + 0.002).to(torch.float16)
    return w, scales


def make_act(seed, m, k, dtype):
    g = H.gen(seed)
    x = torch.randn((m, k), generator=g)
    mask = torch.rand((m, k), generator=g) < 0.01
    x = torch.where(mask, x * 20, x)
    return x.to(H.TORCH_DT[dtype])


@pytest.mark.parametrize("k,n", [(128, 16), (256, 48), (1024, 2048), (5120, 320)])
def test_repack_bit_exact_and_round_trip(ops, oracle, k, n):
    w, _ = make_weight(k + n, k, n)
    p = ops.w4a8_repack_weight(w.cuda())
    np.testing.assert_array_equal(p.cpu().numpy().view(np.uint32), oracle.w4a8_repack_weight(w.numpy().view(np.int8)))
    assert torch.equal(ops.w4a8_unpack_weight(p, k, n).cpu(), w)


def test_repack_rejects_bad_shapes(ops):
    from ksanallm_amd import lib as L
    for k, n in ((100, 16), (128, 24)):
        with pytest.raises(L.KsqError) as e:
            ops.w4a8_repack_weight(torch.zeros((k, n // 2), dtype=torch.uint8, device="cuda"))
        assert e.value.code == 1


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("m,k", [(1, 128), (5, 384), (33, 2048), (130, 5120)])
def test_static_quant_bit_exact(ops, oracle, dtype, per_channel, m, k):
    x = make_act(m * 7 + k, m, k, dtype)
    g = H.gen(m + k)
    scale = (torch.rand(k if per_channel else 1, generator=g) * 0.2 + 0.01).float()
    q, xsum = ops.w4a8_static_quant(x.cuda(), scale.cuda(), per_channel)
    ref = oracle.w4a8_static_quant(H.bits_of(x), scale.numpy(), per_channel, dtype)
    np.testing.assert_array_equal(q.cpu().numpy(), ref)
    np.testing.assert_array_equal(xsum.cpu().numpy().T, oracle.w4a8_group_sums(ref))
    # sums of activations that are quantized already
    np.testing.assert_array_equal(ops.w4a8_group_sums(q).cpu().numpy().T, oracle.w4a8_group_sums(ref))


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
def test_static_quant_per_token_bit_exact(ops, oracle, dtype):
    m, k = 70, 1536
    x = make_act(31, m, k, dtype)
    scale = (torch.rand(m, generator=H.gen(32)) * 0.2 + 0.01).float()
    q, xsum = ops.w4a8_static_quant(x.cuda(), scale.cuda(), per_token=True)
    ref = oracle.w4a8_static_quant(H.bits_of(x), scale.numpy(), False, dtype, per_token=True)
    np.testing.assert_array_equal(q.cpu().numpy(), ref)
    np.testing.assert_array_equal(xsum.cpu().numpy().T, oracle.w4a8_group_sums(ref))


def test_static_quant_boundaries_and_specials(ops, oracle):
    """Every midpoint between neighbouring e4m3 values and its fp32 neighbours, at scale 1; saturation; infinities."""
    codes = np.arange(0, 0x7E, dtype=np.uint8)
    lo, hi = oracle.e4m3_to_f32(codes), oracle.e4m3_to_f32(codes + 1)
    mid = ((lo.astype(np.float64) + hi) / 2).astype(np.float32)
    vals = np.concatenate([mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)), lo,
                           np.float32([448, 449, 464, 465, 1e30, np.inf, 0.0])])
    vals = np.concatenate([vals, -vals])
    pad = (-len(vals)) % 128
    vals = np.concatenate([vals, np.zeros(pad, np.float32)]).reshape(1, -1)
    # fp16 cannot hold all of these; bf16 neither: feed what the type can represent and compare with the oracle on
    # the same bits
    for dtype in (H.F16, H.BF16):
        x = torch.from_numpy(vals).to(H.TORCH_DT[dtype])
        one = torch.ones(1, dtype=torch.float32)
        q, _ = ops.w4a8_static_quant(x.cuda(), one.cuda(), False)
        np.testing.assert_array_equal(q.cpu().numpy(), oracle.w4a8_static_quant(H.bits_of(x), one.numpy(), False, dtype))
    # a scale that makes quotients land between codes
    x = torch.from_numpy(vals).to(torch.float16)
    s = torch.tensor([0.3], dtype=torch.float32)
    q, _ = ops.w4a8_static_quant(x.cuda(), s.cuda(), False)
    np.testing.assert_array_equal(q.cpu().numpy(), oracle.w4a8_static_quant(H.bits_of(x), s.numpy(), False, H.F16))


@pytest.mark.parametrize("out_dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("m", [1, 8, 16, 17, 32, 33, 100, 256])
@pytest.mark.parametrize("n,k", [(2048, 1024), (16, 128), (5120, 5120), (48, 640)])
def test_gemm(ops, oracle, out_dtype, m, n, k):
    if (n, k) == (5120, 5120) and m not in (1, 17, 100, 256):
        pytest.skip("large shape at three token counts")
    w, scales = make_weight(n * 3 + k, k, n)
    x = make_act(m + n + k, m, k, H.BF16)
    in_scale = torch.tensor([0.05], dtype=torch.float32)
    alpha = 0.05 * 0.7
    xq, xsum = ops.w4a8_static_quant(x.cuda(), in_scale.cuda(), False)
    wp = ops.w4a8_repack_weight(w.cuda())
    ref = oracle.w4a8_gemm(xq.cpu().numpy(), w.numpy().view(np.int8), H.bits_of(scales), alpha)
    for rule in H.each_regime(m):  # above 32 tokens: the streaming kernel over 32-token blocks where the problem is small, and the tile kernel
        out = ops.w4a8_gemm(xq, xsum, wp, scales.cuda(), alpha, n, H.TORCH_DT[out_dtype])
        H.check_gemm(out, ref, out_dtype, "w4a8 m=%d n=%d k=%d, small-problem rule %s" % (m, n, k, rule))


@pytest.mark.parametrize("m,n,k", [
    (64, 256, 8192),     # a grid far smaller than the chip: cut along K, partial tiles through the workspace
    (33, 48, 128),       # one k-block, one short column tile
    (130, 2064, 1024),   # N not a multiple of the 256-column tile
    (257, 512, 640),     # M not a multiple of 4: the per-lane form of the group-sum staging
    (300, 1024, 1024),   # 128-token tiles with a half-empty last block
    (1024, 1024, 2048),
    (515, 13328, 512),
    (512, 4352, 256),    # the next three: more than 32 tiles of 256 tokens, the sizes that keep the 256-token tile
    (200, 8704, 256),
    (1024, 2304, 384),
])
@pytest.mark.parametrize("out_dtype", [H.F16, H.BF16])
def test_gemm_tile_kernel(ops, oracle, tile_kernels, out_dtype, m, n, k):
    w, scales = make_weight(n + k + m, k, n)
    x = make_act(m * 3 + n, m, k, H.F16)
    in_scale = torch.tensor([0.04], dtype=torch.float32)
    alpha = 0.04 * 1.3
    xq, xsum = ops.w4a8_static_quant(x.cuda(), in_scale.cuda(), False)
    wp = ops.w4a8_repack_weight(w.cuda())
    out = ops.w4a8_gemm(xq, xsum, wp, scales.cuda(), alpha, n, H.TORCH_DT[out_dtype])
    ref = oracle.w4a8_gemm(xq.cpu().numpy(), w.numpy().view(np.int8), H.bits_of(scales), alpha)
    H.check_gemm(out, ref, out_dtype, "w4a8 tile m=%d n=%d k=%d" % (m, n, k))


@pytest.mark.parametrize("m,n,k", [(3, 8192, 512), (20, 8192, 512), (16, 16384, 256), (32, 16384, 256), (1, 4096, 1024)])
def test_gemm_streaming_kernel_variants(ops, oracle, m, n, k):
    """The streaming kernel's other instantiations: four strips per workgroup with eight wavefronts (n = 8192) and with
    four (n = 16384), one and two 16-token tiles; two strips with eight wavefronts (n = 4096)."""
    w, scales = make_weight(n + k + m, k, n)
    x = make_act(m * 5 + n, m, k, H.BF16)
    in_scale = torch.tensor([0.06], dtype=torch.float32)
    xq, xsum = ops.w4a8_static_quant(x.cuda(), in_scale.cuda(), False)
    out = ops.w4a8_gemm(xq, xsum, ops.w4a8_repack_weight(w.cuda()), scales.cuda(), 0.02, n, torch.bfloat16)
    ref = oracle.w4a8_gemm(xq.cpu().numpy(), w.numpy().view(np.int8), H.bits_of(scales), 0.02)
    H.check_gemm(out, ref, H.BF16, "w4a8 streaming m=%d n=%d k=%d" % (m, n, k))


def test_gemm_workspace_is_checked(ops, tile_kernels):
    from ksanallm_amd import lib as L
    m, n, k = 64, 256, 8192
    need = L.load().ksq_w4a8_workspace_size(m, n, k)
    assert need > 0
    w, scales = make_weight(1, k, n)
    xq = torch.zeros((m, k), dtype=torch.uint8, device="cuda")
    xsum = torch.zeros((k // 128, m), dtype=torch.float32, device="cuda")
    wp = ops.w4a8_repack_weight(w.cuda())
    with pytest.raises(L.KsqError) as e:
        ops.w4a8_gemm(xq, xsum, wp, scales.cuda(), 1.0, n, workspace=torch.empty(256, dtype=torch.uint8, device="cuda"))
    assert e.value.code == 3
    out = ops.w4a8_gemm(xq, xsum, wp, scales.cuda(), 1.0, n)
    assert torch.all(out == 0)


def test_gemm_full_size_properties(ops):
    """At the reference's own performance shape (n = 25600, k = 5120; finegrained_mixed_dtype_gemm_thop_test.cu:312-321)
    with 4096 tokens, where the oracle would take minutes:
      * the tile kernel agrees with the streaming kernel run on 32-token chunks of the same rows (same products and
        fp32 partial sums per group, summed in another order: one unit in the last place of the output at most, plus
        what reordering an fp32 sum of forty terms of magnitude ~10 can move, which matters for results near zero);
      * permuting the tokens permutes the output rows bit for bit;
      * zero activations give zeros."""
    m, n, k = 4096, 25600, 5120
    w, scales = make_weight(7, k, n)
    x = make_act(8, m, k, H.BF16)
    in_scale = torch.tensor([0.05], dtype=torch.float32)
    xq, xsum = ops.w4a8_static_quant(x.cuda(), in_scale.cuda(), False)
    wp = ops.w4a8_repack_weight(w.cuda())
    sc = scales.cuda()
    out = ops.w4a8_gemm(xq, xsum, wp, sc, 0.03, n)
    for r0 in (0, 2016, 4064):
        rows = slice(r0, r0 + 32)
        part = ops.w4a8_gemm(xq[rows].contiguous(), xsum[:, rows].contiguous(), wp, sc, 0.03, n)
        a, b = out[rows].float(), part.float()
        ulp = torch.from_numpy(H.ulp(b.cpu().numpy(), H.BF16)).cuda()
        assert bool(torch.all((a - b).abs() <= ulp + 5e-5)), "rows %d..: %g" % (r0, float((a - b).abs().max()))
    perm = torch.randperm(m, generator=H.gen(9)).cuda()
    out_p = ops.w4a8_gemm(xq[perm].contiguous(), xsum[:, perm].contiguous(), wp, sc, 0.03, n)
    assert torch.equal(out_p, out[perm])
    zq = torch.zeros_like(xq)
    assert torch.all(ops.w4a8_gemm(zq, ops.w4a8_group_sums(zq), wp, sc, 0.03, n) == 0)


def test_gemm_extreme_codes_and_sums(ops, oracle):
    """All weights -8 (the code that needs the offset term most) and all +7, activations of one sign: the offset term
    -8 * sum(x) is as large as it gets against the result."""
    m, n, k = 16, 64, 1024
    for byte in (0x88, 0x77, 0x00):
        w = torch.full((k, n // 2), byte, dtype=torch.uint8)
        scales = torch.full((k // 128, n), 0.01, dtype=torch.float16)
        x = (torch.rand((m, k), generator=H.gen(byte)) * 3 + 1).to(torch.float16)
        one = torch.ones(1, dtype=torch.float32)
        xq, xsum = ops.w4a8_static_quant(x.cuda(), one.cuda(), False)
        out = ops.w4a8_gemm(xq, xsum, ops.w4a8_repack_weight(w.cuda()), scales.cuda(), 1.0, n, torch.float16)
        ref = oracle.w4a8_gemm(xq.cpu().numpy(), w.numpy().view(np.int8), H.bits_of(scales), 1.0)
        if byte == 0x00:
            assert torch.all(out == 0)
        else:
            H.check_gemm(out, ref, H.F16, "w4a8 constant weights 0x%02x" % byte)


def test_gemm_meets_the_reference_tests_own_tolerance(ops, oracle):
    """The reference's check (finegrained_mixed_dtype_gemm_thop_test.cu:140-158, 186-210): |out - ref| <=
    1.5 * max|ref| / 8 against a bf16 matmul of the dequantized weights, at its shape (512, 2048, 1024)."""
    m, n, k = 512, 2048, 1024
    g = H.gen(42)
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    w, _ = make_weight(42, k, n)
    scales = torch.rand((k // 128, n), generator=g).to(torch.float16)
    alpha = float(torch.rand(1, generator=g))
    xq = x.cuda().to(torch.float8_e4m3fn).view(torch.uint8)  # the test casts the activations directly
    out = ops.w4a8_gemm(xq, ops.w4a8_group_sums(xq), ops.w4a8_repack_weight(w.cuda()), scales.cuda(), alpha, n)
    wt = torch.from_numpy(oracle.w4a8_unpack_int4(w.numpy().view(np.int8))).cuda().to(torch.bfloat16)
    wref = wt * scales.cuda().repeat_interleave(128, 0).to(torch.bfloat16)
    ref = ((x.cuda() * alpha).to(torch.bfloat16) @ wref).float()
    atol = float(ref.abs().max()) / 8 * 1.5
    assert float((out.float() - ref).abs().max()) <= atol


@pytest.mark.parametrize("m,n,k", [(1, 2048, 1024), (16, 48, 640), (17, 8192, 512), (32, 16, 128),     # streaming kernel
                                   (33, 48, 128), (130, 2064, 1024), (257, 512, 640), (300, 1024, 1024),  # 128-token tiles
                                   (1024, 2304, 384)])
@pytest.mark.parametrize("out_dtype", [H.F16, H.BF16])
def test_gemm_group_64(ops, oracle, out_dtype, m, n, k):
    """Scale groups of 64: sums per 64 channels bit-exact, the GEMM (both kernels) against the oracle; and with scales
    equal in both halves of every 128 channels the result has the bits of the group-128 launch."""
    g = H.gen(m + n + k)
    w = torch.randint(0, 256, (k, n // 2), generator=g, dtype=torch.uint8)
    s64 = (torch.rand((k // 64, n), generator=g) * 0.02 + 0.002).to(torch.float16)
    x = make_act(m * 7 + k, m, k, H.BF16)
    in_scale = torch.tensor([0.05], dtype=torch.float32)
    xq, xsum = ops.w4a8_static_quant(x.cuda(), in_scale.cuda(), False, group=64)
    np.testing.assert_array_equal(xsum.cpu().numpy().T, oracle.w4a8_group_sums(xq.cpu().numpy(), 64))
    np.testing.assert_array_equal(ops.w4a8_group_sums(xq, 64).cpu().numpy(), xsum.cpu().numpy())
    wp = ops.w4a8_repack_weight(w.cuda())
    ref = oracle.w4a8_gemm(xq.cpu().numpy(), w.numpy().view(np.int8), H.bits_of(s64), 0.03, group=64)
    s128 = s64[0::2].contiguous()
    same = s128.repeat_interleave(2, 0).contiguous()
    for rule in H.each_regime(m):
        out = ops.w4a8_gemm(xq, xsum, wp, s64.cuda(), 0.03, n, H.TORCH_DT[out_dtype], group=64)
        H.check_gemm(out, ref, out_dtype, "w4a8 g64 m=%d n=%d k=%d, small-problem rule %s" % (m, n, k, rule))
        a = ops.w4a8_gemm(xq, xsum, wp, same.cuda(), 0.03, n, H.TORCH_DT[out_dtype], group=64)
        b = ops.w4a8_gemm(xq, ops.w4a8_group_sums(xq), wp, s128.cuda(), 0.03, n, H.TORCH_DT[out_dtype])
        H.check_gemm(a, b.float().cpu().numpy(), out_dtype, "w4a8 g64 against g128")


def test_gemm_rejects_what_it_does_not_do(ops):
    from ksanallm_amd import lib as L
    lib = L.load()
    z = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    p = z.data_ptr()
    # group 32
    assert lib.ksq_w4a8_gemm(p, p, p, p, 1.0, p, 1, 16, 128, 32, L.BF16, None, 0, None) == 2
    # n not a multiple of 16, k not of 128
    assert lib.ksq_w4a8_gemm(p, p, p, p, 1.0, p, 1, 24, 128, 128, L.BF16, None, 0, None) == 1
    assert lib.ksq_w4a8_gemm(p, p, p, p, 1.0, p, 1, 16, 100, 128, L.BF16, None, 0, None) == 1
    assert lib.ksq_w4a8_gemm(None, p, p, p, 1.0, p, 1, 16, 128, 128, L.BF16, None, 0, None) == 1
    assert b"ksq_w4a8_gemm" in lib.ksq_last_error_string()
    # m = 0 is a no-op
    assert lib.ksq_w4a8_gemm(p, p, p, p, 1.0, p, 0, 16, 128, 128, L.BF16, None, 0, None) == 0
