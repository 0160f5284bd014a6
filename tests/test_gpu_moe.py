"""MoE path: expert-offset/permutation build (bit-exact), grouped W4A16 GEMM, silu*mul, top-k sum, whole block."""
import numpy as np
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from ksanallm_amd import ops
    return ops


def test_align_worked_example(ops):
    ids = torch.tensor([0, 1, 2, 1, 2, 3, 0, 3, 4], dtype=torch.int32).cuda()
    s, e, npp = ops.moe_align_block_size(ids, 5, 4)
    P = 9
    assert s.cpu().tolist()[:20] == [0, 6, P, P, 1, 3, P, P, 2, 4, P, P, 5, 7, P, P, 8, P, P, P]
    assert npp.item() == 20 and e.cpu().tolist()[:5] == [0, 1, 2, 3, 4]


@pytest.mark.parametrize("E,bm,T,topk", [(256, 16, 1, 8), (256, 16, 64, 8), (256, 32, 512, 8), (256, 64, 4096, 8),
                                         (8, 4, 3, 2), (1000, 16, 77, 6), (60, 16, 32768, 4)])
def test_align_bit_exact(ops, oracle, E, bm, T, topk):
    g = H.gen(E + T)
    logits = torch.randn((T, E), generator=g)
    ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1).indices.to(torch.int32)
    s, e, npp = ops.moe_align_block_size(ids.cuda(), E, bm)
    so, eo, nppo = oracle.moe_align(ids.numpy(), E, bm)
    assert npp.item() == nppo
    np.testing.assert_array_equal(s.cpu().numpy(), so)
    nb = nppo // bm
    np.testing.assert_array_equal(e.cpu().numpy()[:nb], eo[:nb])


def test_align_out_of_range_ids_dropped(ops, oracle):
    ids = torch.tensor([0, 7, -1, 2, 300, 2], dtype=torch.int32)
    s, e, npp = ops.moe_align_block_size(ids.cuda(), 4, 2)
    so, eo, nppo = oracle.moe_align(ids.numpy(), 4, 2)
    assert npp.item() == nppo
    np.testing.assert_array_equal(s.cpu().numpy(), so)


@pytest.mark.parametrize("numel,E,bm", [(1, 256, 16), (8, 256, 16), (63, 5, 32), (64, 1, 16), (65, 192, 128), (256, 7, 16),
                                        (257, 64, 256), (1000, 12, 32), (1024, 192, 16), (1024, 1000, 16)])
def test_align_few_ids(ops, oracle, numel, E, bm):
    # decode batches (one id per thread, counters in LDS): every wavefront count around 64, one expert taking all ids,
    # ids outside [0, E), and a shape whose counters do not fit and falls back to the general kernel
    g = H.gen(7 * numel + E)
    ids = torch.randint(-2, E + 2, (numel,), generator=g, dtype=torch.int32)
    s, e, npp = ops.moe_align_block_size(ids.cuda(), E, bm)
    so, eo, nppo = oracle.moe_align(ids.numpy(), E, bm)
    assert npp.item() == nppo
    np.testing.assert_array_equal(s.cpu().numpy(), so)
    nb = nppo // bm
    np.testing.assert_array_equal(e.cpu().numpy()[:nb], eo[:nb])


@pytest.mark.parametrize("numel,E,bm", [(2048, 7, 128), (2049, 4096, 16), (33333, 300, 32), (70001, 1, 128)])
def test_align_many_ids_ragged(ops, oracle, numel, E, bm):
    # the sort over several workgroups: ragged chunk ends, ids outside [0, E), one expert, the largest expert count
    g = H.gen(numel + E)
    ids = torch.randint(-3, E + 3, (numel,), generator=g, dtype=torch.int32)
    s, e, npp = ops.moe_align_block_size(ids.cuda(), E, bm)
    so, eo, nppo = oracle.moe_align(ids.numpy(), E, bm)
    assert npp.item() == nppo
    np.testing.assert_array_equal(s.cpu().numpy(), so)
    nb = nppo // bm
    np.testing.assert_array_equal(e.cpu().numpy()[:nb], eo[:nb])


@pytest.mark.parametrize("T,E,topk", [(1, 256, 8), (77, 256, 8), (5, 60, 4), (9, 1000, 6)])
def test_topk_softmax(ops, oracle, T, E, topk):
    g = H.gen(T + E)
    logits = torch.randn((T, E), generator=g)
    logits[0, :4] = logits[0, 7]  # ties
    for norm in (False, True):
        w, ids = ops.moe_topk_softmax(logits.cuda(), topk, norm, 2.5)
        wo, io = oracle.moe_topk_softmax(logits.numpy(), topk, norm, 2.5, 2)
        np.testing.assert_array_equal(ids.cpu().numpy(), io)
        np.testing.assert_allclose(w.cpu().numpy(), wo, rtol=2e-6, atol=1e-9)
    lb = logits.to(torch.bfloat16)
    w, ids = ops.moe_topk_softmax(lb.cuda(), topk)
    wo, io = oracle.moe_topk_softmax(H.bits_of(lb), topk, False, 1.0, H.BF16)
    np.testing.assert_array_equal(ids.cpu().numpy(), io)


def _check_routing(w, ids, wo, io, choose_gap_ok):
    """ids equal as sets per token; where they differ (expf on the GPU and on the host may round differently and swap
    two near-equal scores) the two experts' weights must agree to 3e-4, the reference test's own allowance."""
    w, ids = w.cpu().numpy(), ids.cpu().numpy()
    order, order_o = np.argsort(ids, -1), np.argsort(io, -1)
    ids_s, io_s = np.take_along_axis(ids, order, -1), np.take_along_axis(io, order_o, -1)
    w_s, wo_s = np.take_along_axis(w, order, -1), np.take_along_axis(wo, order_o, -1)
    diff = ids_s != io_s
    assert diff.mean() <= choose_gap_ok
    np.testing.assert_allclose(w_s[~diff], wo_s[~diff], rtol=2e-5, atol=1e-8)
    np.testing.assert_allclose(np.sort(w, -1), np.sort(wo, -1), atol=3e-4)


@pytest.mark.parametrize("T,E,topk,groups,topk_group,scoring,use_bias,renorm", [
    (2048, 256, 8, 8, 4, "sigmoid", True, True),     # DeepSeek-V3, the reference test's first config
    (2048, 128, 4, 4, 2, "sigmoid", True, True),     # its second config
    (77, 160, 6, 8, 3, "softmax", False, False),     # DeepSeek-V2
    (5, 64, 6, 1, 1, "sigmoid", False, True),
    (9, 1000, 6, 1, 1, "softmax", False, True),
    (1, 256, 8, 8, 4, "sigmoid", True, True),
    (33, 512, 6, 8, 3, "sigmoid", True, True),       # more than 256 experts with real groups: the 16-slots-per-lane form
])
def test_grouped_topk(ops, oracle, T, E, topk, groups, topk_group, scoring, use_bias, renorm):
    g = H.gen(T + E)
    logits = torch.rand((T, E), generator=g) * 1.98 - 0.99
    bias = (torch.rand(E, generator=g) * 0.009 - 0.01) if use_bias else None
    for dtype, lt in ((oracle.F32, logits), (H.BF16, logits.to(torch.bfloat16)), (H.F16, logits.to(torch.float16))):
        w, ids = ops.moe_grouped_topk(lt.cuda(), topk, groups, topk_group, scoring, None if bias is None else bias.cuda(),
                                      renorm, 2.5)
        src = lt.numpy() if dtype == oracle.F32 else H.bits_of(lt)
        wo, io = oracle.moe_grouped_topk(src, None if bias is None else bias.numpy(), topk, groups, topk_group,
                                         scoring == "sigmoid", renorm, 2.5, dtype)
        # 16-bit logits tie often (few distinct values): ties resolve identically (lower id), so ids still match
        _check_routing(w, ids, wo, io, 1e-3)
        if renorm:
            np.testing.assert_allclose(w.cpu().numpy().sum(-1), 2.5, rtol=1e-5)


# the HIP router against the reference's own host implementation (oracle/_ref, built beforehand from the reference tree)
@pytest.mark.parametrize("T,E,topk,groups,topk_group", [(2048, 256, 8, 8, 4), (333, 128, 4, 4, 2)])
def test_grouped_topk_vs_reference_host_code(ops, oracle, T, E, topk, groups, topk_group):
    g = H.gen(3 * T + E)
    logits = torch.rand((T, E), generator=g) * 1.98 - 0.99
    bias = torch.rand(E, generator=g) * 0.009 - 0.01
    ref = oracle.ref_grouped_topk(logits.numpy(), bias.numpy(), topk, groups, topk_group, 2.5)
    if ref is None:
        pytest.skip("oracle/_ref is not built")
    rw, ri = ref
    w, ids = ops.moe_grouped_topk(logits.cuda(), topk, groups, topk_group, "sigmoid", bias.cuda(), True, 2.5)
    w, ids = w.cpu().numpy(), ids.cpu().numpy()
    swapped = 0
    for t in range(T):
        if sorted(ids[t].tolist()) != sorted(ri[t].tolist()):
            swapped += 1      # GPU and host expf may order two near-equal scores differently
            continue
        mine = dict(zip(ids[t].tolist(), w[t].tolist()))
        for e, x in zip(ri[t].tolist(), rw[t].tolist()):
            assert abs(mine[e] - x) <= 3e-4, (t, e, mine[e], x)
    assert swapped <= T // 200, swapped


def test_grouped_topk_matches_plain_softmax_router(ops):
    g = H.gen(5)
    logits = torch.randn((33, 256), generator=g).cuda()
    w0, i0 = ops.moe_topk_softmax(logits, 8, True, 2.5)
    w1, i1 = ops.moe_grouped_topk(logits, 8, 1, 1, "softmax", None, True, 2.5)
    assert torch.equal(i0, i1)
    torch.testing.assert_close(w0, w1, rtol=1e-6, atol=0)


def test_grouped_topk_rejects_bad_arguments(ops):
    from ksanallm_amd import lib as L
    x = torch.zeros((2, 256), device="cuda")
    for kw in (dict(num_expert_group=7), dict(num_expert_group=8, topk_group=9), dict(num_expert_group=128, topk_group=1),
               dict(top_k=40), dict(num_expert_group=64, topk_group=1, top_k=8)):
        args = dict(top_k=8, num_expert_group=8, topk_group=4)
        args.update(kw)
        with pytest.raises(L.KsqError) as e:
            ops.moe_grouped_topk(x, args["top_k"], args["num_expert_group"], args["topk_group"], "sigmoid")
        assert e.value.code == 1
    with pytest.raises(ValueError):
        ops.moe_grouped_topk(x, 8, 8, 4, "tanh")


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
def test_silu_mul_and_sum(ops, oracle, dtype):
    g = H.gen(3)
    x = (torch.randn((37, 512), generator=g) * 3).to(H.TORCH_DT[dtype])
    out = ops.silu_and_mul(x.cuda())
    ref = oracle.from_bits(oracle.silu_mul(H.bits_of(x), dtype), dtype)
    # expf on the GPU and on the host may differ in the last bit before rounding to T
    got = out.float().cpu().numpy()
    assert np.abs(got - ref).max() <= np.abs(ref).max() * 2.0 ** (-7 if dtype == H.BF16 else -10)
    assert (got == ref).mean() > 0.99
    y = torch.randn((19, 8, 256), generator=g).to(H.TORCH_DT[dtype])
    got = ops.moe_sum(y.cuda())
    ref = oracle.moe_sum(H.bits_of(y), dtype)
    np.testing.assert_array_equal(H.bits_of(got.cpu()), ref)


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("T,E,topk,hidden,inter,bm", [(1, 8, 2, 256, 128, 16), (5, 16, 4, 512, 256, 16), (70, 8, 2, 384, 80 * 16, 32),
                                                      (33, 256, 8, 7168, 2048, 16), (300, 16, 4, 256, 16, 32),
                                                      (300, 6, 3, 256, 80 * 16, 128), (700, 4, 2, 384, 1024, 256),
                                                      (130, 2, 1, 256, 16, 256), (520, 8, 2, 512, 2048, 128)])
def test_gate_up_with_silu_in_the_epilogue_equals_the_two_launches(ops, dtype, T, E, topk, hidden, inter, bm):
    """ksq_moe_w4a16_gate_up_silu against ksq_moe_w4a16_gemm + ksq_silu_mul on the same inputs: the same bits."""
    from ksanallm_amd import lib as L
    g = H.gen(8800 + T + inter)
    td = H.TORCH_DT[dtype]
    w13 = torch.randint(0, 256, (E, 2 * inter, hidden // 2), generator=g, dtype=torch.uint8)
    s13 = H.uniform(g, (E, 2 * inter, hidden // 128), 0.002, 0.01, dtype)
    x = torch.randn((T, hidden), generator=g).to(td).cuda()
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)]).to(torch.int32).cuda()
    wp = ops.repack_weight(w13.cuda(), L.SRC_MOE_NK, E, hidden, 2 * inter)
    sp = ops.repack_scales(s13.cuda(), L.SCALE_NG, E, hidden, 2 * inter, 128)
    numel = T * topk
    s, e, npp = ops.moe_align_block_size(ids, E, bm)
    two = ops.silu_and_mul(ops.moe_w4a16_gemm(x, wp, sp, None, s, e, npp, numel, topk, E, 2 * inter, hidden, 128, bm))
    one = ops.moe_w4a16_gate_up_silu(x, wp, sp, s, e, npp, numel, topk, E, 2 * inter, hidden, 128, bm)
    torch.cuda.synchronize()
    assert torch.equal(one.view(torch.int16), two.view(torch.int16))
    with pytest.raises(L.KsqError) as err:   # a block size that no kernel has
        ops.moe_w4a16_gate_up_silu(x, wp, sp, s, e, npp, numel, topk, E, 2 * inter, hidden, 128, 64)
    assert err.value.code == 2


def make_moe(oracle, seed, E, hidden, inter, T, topk, group, dtype):
    g = H.gen(seed)
    td = H.TORCH_DT[dtype]
    w13 = torch.randint(0, 256, (E, 2 * inter, hidden // 2), generator=g, dtype=torch.uint8)
    w2 = torch.randint(0, 256, (E, hidden, inter // 2), generator=g, dtype=torch.uint8)
    s13 = H.uniform(g, (E, 2 * inter, hidden // group), 0.002, 0.01, dtype)
    s2 = H.uniform(g, (E, hidden, inter // group), 0.002, 0.01, dtype)
    x = torch.randn((T, hidden), generator=g).to(td)
    logits = torch.randn((T, E), generator=g)
    tw, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
    return dict(w13=w13, w2=w2, s13=s13, s2=s2, x=x, ids=ids.to(torch.int32), tw=tw.float().contiguous(), E=E,
                hidden=hidden, inter=inter, T=T, topk=topk, group=group, dtype=dtype)


def pack_moe(ops, d):
    from ksanallm_amd import lib as L
    E, H_, I, g = d["E"], d["hidden"], d["inter"], d["group"]
    return (ops.repack_weight(d["w13"].cuda(), L.SRC_MOE_NK, E, H_, 2 * I),
            ops.repack_scales(d["s13"].cuda(), L.SCALE_NG, E, H_, 2 * I, g),
            ops.repack_weight(d["w2"].cuda(), L.SRC_MOE_NK, E, I, H_),
            ops.repack_scales(d["s2"].cuda(), L.SCALE_NG, E, I, H_, g))


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("T,bm", [(1, 16), (5, 16), (64, 16), (64, 32), (64, 128), (300, 128), (512, 128), (300, 256), (700, 256)])
def test_grouped_gemm_stages(ops, oracle, dtype, T, bm):
    d = make_moe(oracle, 5000 + T, 16, 256, 128, T, 4, 128, dtype)
    w13p, s13p, w2p, s2p = pack_moe(ops, d)
    numel = T * d["topk"]
    s, e, npp = ops.moe_align_block_size(d["ids"].cuda(), d["E"], bm)
    c1 = ops.moe_w4a16_gemm(d["x"].cuda(), w13p, s13p, None, s, e, npp, numel, d["topk"], d["E"], 2 * d["inter"],
                            d["hidden"], 128, bm)
    ref1 = oracle.moe_w4a16_gemm(H.bits_of(d["x"]), d["w13"].numpy(), H.bits_of(d["s13"]), d["ids"].numpy(),
                                 d["tw"].numpy(), d["topk"], 128, False, dtype)
    H.check_gemm(c1, ref1, dtype, "moe gemm1", weights_rounded=bm == 128)
    c2 = ops.silu_and_mul(c1)
    c3 = ops.moe_w4a16_gemm(c2, w2p, s2p, d["tw"].cuda().reshape(-1), s, e, npp, numel, 1, d["E"], d["hidden"],
                            d["inter"], 128, bm)
    ref3 = oracle.moe_w4a16_gemm(H.bits_of(c2.cpu()), d["w2"].numpy(), H.bits_of(d["s2"]), d["ids"].numpy(),
                                 d["tw"].numpy(), 1, 128, True, dtype)
    H.check_gemm(c3, ref3, dtype, "moe gemm2", weights_rounded=bm == 128)


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("bm", [128, 256])
def test_grouped_tile_kernel_every_count_of_live_row_tiles(ops, oracle, dtype, bm):
    """The tile kernel has an instance of its main loop per number of row tiles that hold rows: experts with
    16c - 5 rows for c = 4..16, and one with 3 rows, meet every instance of the 256-row form (and, cut into 128-row
    blocks, of the 128-row form)."""
    rows = [16 * c - 5 for c in range(4, 17)] + [3]
    E, T = len(rows), sum(rows)
    d = make_moe(oracle, 5900 + bm, E, 256, 128, T, 1, 128, dtype)
    ids = torch.cat([torch.full((r,), e, dtype=torch.int32) for e, r in enumerate(rows)])
    ids = ids[torch.randperm(T, generator=H.gen(77))].reshape(T, 1).contiguous()
    w13p, s13p, _, _ = pack_moe(ops, d)
    s, e, npp = ops.moe_align_block_size(ids.cuda(), E, bm)
    c1 = ops.moe_w4a16_gemm(d["x"].cuda(), w13p, s13p, None, s, e, npp, T, 1, E, 2 * d["inter"], d["hidden"], 128, bm)
    ref1 = oracle.moe_w4a16_gemm(H.bits_of(d["x"]), d["w13"].numpy(), H.bits_of(d["s13"]), ids.numpy(), d["tw"].numpy(), 1,
                                 128, False, dtype)
    H.check_gemm(c1, ref1, dtype, "grouped tile kernel, %d-row blocks" % bm, weights_rounded=True)


@pytest.mark.parametrize("T", [1, 64, 2048])
def test_moe_block_deepseek_shape(ops, oracle, T):
    """256 experts, hidden 7168, inter 2048, top-8; weights for all experts are generated but only touched ones
    matter.  Scaled to 32 experts' worth of memory on the host by reusing expert slabs."""
    E, hidden, inter, topk = 256, 7168, 2048, 8
    base = make_moe(oracle, 5100 + T, 8, hidden, inter, T, topk, 128, H.BF16)
    rep = E // 8
    d = dict(base)
    d["E"] = E
    for k in ("w13", "w2", "s13", "s2"):
        d[k] = base[k].repeat((rep, 1, 1))
    g = H.gen(77 + T)
    logits = torch.randn((T, E), generator=g)
    tw, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
    d["ids"], d["tw"] = ids.to(torch.int32), tw.float().contiguous()
    w13p, s13p, w2p, s2p = pack_moe(ops, d)
    out = ops.fused_moe_w4a16(d["x"].cuda(), w13p, s13p, w2p, s2p, d["ids"].cuda(), d["tw"].cuda(), E, hidden, inter,
                              128)
    ref = oracle.moe_forward(H.bits_of(d["x"]), d["w13"].numpy(), H.bits_of(d["s13"]), d["w2"].numpy(),
                             H.bits_of(d["s2"]), d["ids"].numpy(), d["tw"].numpy(), 128, H.BF16)
    ref = oracle.from_bits(ref, H.BF16)
    # intermediate tensors are rounded to bf16 at three places in both implementations, so the end-to-end
    # comparison carries those roundings: rel-L2 stays the gate, the absolute bound is the GEMM one
    # T = 2048 runs both GEMMs through the MFMA tile kernel, which rounds every dequantized weight to bf16 (each GEMM
    # on its own is held to 5e-3 in test_grouped_gemm_stages); two such GEMMs in a row compound to sqrt(2) of that
    rounded = T * topk // E >= 64
    H.check_gemm(out, ref, H.BF16, "moe block T=%d" % T, weights_rounded=rounded,
                 rel_l2_max=5e-3 * (2 ** 0.5 if rounded else 1.0))


@pytest.mark.parametrize("T", [512, 4096])
def test_moe_block_benchmark_token_counts(ops, oracle, T):
    """The benchmark's two larger token counts at its own shapes (256 experts, hidden 7168, inter 2048, top-8): the GPU
    runs the whole block, the oracle the first 8 and the last 4 tokens of it (a token's output depends on its own
    row, experts and routing weights only)."""
    E, hidden, inter, topk = 256, 7168, 2048, 8
    base = make_moe(oracle, 5200 + T, 8, hidden, inter, T, topk, 128, H.BF16)
    rep = E // 8
    d = dict(base)
    d["E"] = E
    for k in ("w13", "w2", "s13", "s2"):
        d[k] = base[k].repeat((rep, 1, 1))
    logits = torch.randn((T, E), generator=H.gen(78 + T))
    tw, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
    d["ids"], d["tw"] = ids.to(torch.int32), tw.float().contiguous()
    w13p, s13p, w2p, s2p = pack_moe(ops, d)
    out = ops.fused_moe_w4a16(d["x"].cuda(), w13p, s13p, w2p, s2p, d["ids"].cuda(), d["tw"].cuda(), E, hidden, inter,
                              128)
    from ksanallm_amd import lib as L
    rounded = L.load().ksq_moe_block_m(T * topk, E) >= 128
    for sel in (slice(0, 8), slice(T - 4, T)):
        ref = oracle.moe_forward(H.bits_of(d["x"][sel]), d["w13"].numpy(), H.bits_of(d["s13"]), d["w2"].numpy(),
                                 H.bits_of(d["s2"]), d["ids"][sel].contiguous().numpy(), d["tw"][sel].contiguous().numpy(),
                                 128, H.BF16)
        H.check_gemm(out[sel], oracle.from_bits(ref, H.BF16), H.BF16, "moe block T=%d tokens %s" % (T, sel),
                     weights_rounded=rounded, rel_l2_max=5e-3 * (2 ** 0.5 if rounded else 1.0))


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
def test_silu_over_every_input_of_the_type(ops, dtype):
    """silu(g) * 1 for every finite 16-bit g, against the correctly rounded value (float64 silu rounded to T): the
    kernels' one definition of the activation (hardware base-2 exponential, a division, a multiply) may differ from it
    by one unit in the last place and no more, in a small share of the inputs - the figure the design notes quote."""
    td = H.TORCH_DT[dtype]
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    g = bits.view(td)
    g = g[torch.isfinite(g.float())]
    n = g.numel()
    pad = (-n) % 128
    g = torch.cat([g, torch.zeros(pad, dtype=td)])
    x = torch.cat([g.view(-1, 128), torch.ones((g.numel() // 128, 128), dtype=td)], dim=1).contiguous()   # [rows, 2 * 128]: gate | up
    y = ops.silu_and_mul(x.cuda()).cpu().view(-1)[:n]
    g64 = g[:n].double()
    exact = (g64 / (1.0 + torch.exp(-g64))).to(td)
    yi, ei = y.view(torch.int16).int(), exact.view(torch.int16).int()
    # distance in units of the last place, on the ordered integer line of the type's bit patterns
    key = lambda v: torch.where(v < 0, -(v & 0x7fff), v)
    d = (key(yi) - key(ei)).abs()
    # results below 2^-100 (bf16 has fp32's exponent range; exp overflows first) only have to be that small as well
    tiny = (exact.float().abs() < 2.0 ** -100) & (y.float().abs() < 2.0 ** -100)
    d = torch.where(tiny, torch.zeros_like(d), d)
    assert int(d.max()) <= 1, int(d.max())
    share = float((d > 0).float().mean())
    assert share < 0.02, share
    print("silu %s: %d of %d inputs one unit off the correctly rounded value (%.3f %%)" % (td, int((d > 0).sum()), n, 100 * share))


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("T,E,topk,hidden,inter", [(1, 16, 4, 256, 128), (2, 16, 8, 512, 256), (3, 8, 2, 384, 128), (8, 16, 4, 256, 384),
                                                   (1, 256, 8, 7168, 2048)])
def test_few_tokens_without_alignment_and_with_the_sum_in_the_second_gemm(ops, oracle, dtype, T, E, topk, hidden, inter):
    """A handful of slots: the first GEMM with every slot a block of its own (sorted_ids NULL, the router's ids as they
    are) gives the bits of the aligned form; the second GEMM with the sum over top-k in it agrees with the oracle's
    block (its fp32 sum is rounded once where the reference rounds every expert's share first)."""
    from ksanallm_amd import lib as L
    distinct = min(E, 8)
    base = make_moe(oracle, 5300 + T + hidden, distinct, hidden, inter, T, topk, 128, dtype)
    d = dict(base)
    d["E"] = E
    for k in ("w13", "w2", "s13", "s2"):
        d[k] = base[k].repeat((E // distinct, 1, 1))
    logits = torch.randn((T, E), generator=H.gen(79 + T))
    tw, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
    d["ids"], d["tw"] = ids.to(torch.int32).contiguous(), tw.float().contiguous()
    w13p, s13p, w2p, s2p = pack_moe(ops, d)
    numel = T * topk
    x, idf, twf = d["x"].cuda(), d["ids"].cuda().reshape(-1), d["tw"].cuda().reshape(-1)
    lib = L.load()
    stream = torch.cuda.current_stream().cuda_stream
    td = H.TORCH_DT[dtype]
    # first GEMM + activation: every slot its own block, against the aligned form
    s, e, npp = ops.moe_align_block_size(d["ids"].cuda(), E, 16)
    want = ops.moe_w4a16_gate_up_silu(x, w13p, s13p, s, e, npp, numel, topk, E, 2 * inter, hidden, 128, 16)
    c2 = torch.full((numel, inter), float("nan"), dtype=td, device="cuda")
    L.check(lib.ksq_moe_w4a16_gate_up_silu(c2.data_ptr(), x.data_ptr(), w13p.data_ptr(), s13p.data_ptr(), None, None,
                                           idf.data_ptr(), None, numel, topk, E, 2 * inter, hidden, 128, 16, dtype, stream))
    assert torch.equal(c2.view(torch.int16), want.view(torch.int16))
    # plain grouped GEMM in the same form (second GEMM without the sum)
    want3 = ops.moe_w4a16_gemm(c2, w2p, s2p, twf, s, e, npp, numel, 1, E, hidden, inter, 128, 16)
    c3 = torch.full((numel, hidden), float("nan"), dtype=td, device="cuda")
    L.check(lib.ksq_moe_w4a16_gemm(c3.data_ptr(), c2.data_ptr(), w2p.data_ptr(), s2p.data_ptr(), None, twf.data_ptr(), None,
                                   idf.data_ptr(), None, numel, 1, E, hidden, inter, 128, 16, dtype, stream))
    assert torch.equal(c3.view(torch.int16), want3.view(torch.int16))
    # second GEMM with the sum in it, and the whole block through the wrapper, against the oracle
    out = torch.full((T, hidden), float("nan"), dtype=td, device="cuda")
    L.check(lib.ksq_moe_w4a16_down_sum(out.data_ptr(), c2.data_ptr(), w2p.data_ptr(), s2p.data_ptr(), twf.data_ptr(),
                                       idf.data_ptr(), T, topk, E, hidden, inter, 128, dtype, stream))
    # the oracle of this launch: the second GEMM's fp32 rows (routing weight applied) of the same activations, summed
    # over top-k without the rounding to T in between
    rows = oracle.moe_w4a16_gemm(H.bits_of(c2.cpu()), d["w2"].numpy(), H.bits_of(d["s2"]), d["ids"].numpy(), d["tw"].numpy(),
                                 1, 128, True, dtype)
    H.check_gemm(out, rows.reshape(T, topk, hidden).astype(np.float64).sum(1).astype(np.float32), dtype, "down + sum T=%d" % T)
    # and the reference's own sequence (every expert's share rounded to T, then summed in T): the block's rel-L2 bar
    ref = oracle.from_bits(oracle.moe_forward(H.bits_of(d["x"]), d["w13"].numpy(), H.bits_of(d["s13"]), d["w2"].numpy(),
                                              H.bits_of(d["s2"]), d["ids"].numpy(), d["tw"].numpy(), 128, dtype), dtype)
    H.check_gemm(out, ref, dtype, "few-token block T=%d" % T, weights_rounded=True,
                 rel_l2_max=5e-3 + 2.0 ** (-8 if dtype == H.BF16 else -11) * topk ** 0.5)
    if T <= ops.FEW_TOKENS:
        whole = ops.fused_moe_w4a16(x, w13p, s13p, w2p, s2p, d["ids"].cuda(), d["tw"].cuda(), E, hidden, inter, 128)
        assert torch.equal(whole.view(torch.int16), out.view(torch.int16))


def test_few_tokens_form_drops_ids_outside_the_experts_and_rejects_what_it_cannot_do(ops, oracle):
    from ksanallm_amd import lib as L
    E, topk, hidden, inter, T = 8, 4, 256, 128, 2
    d = make_moe(oracle, 5350, E, hidden, inter, T, topk, 128, H.BF16)
    w13p, s13p, w2p, s2p = pack_moe(ops, d)
    ids = d["ids"].clone()
    ids[0, 1] = E + 3              # an id the alignment would drop
    ids[1, 2] = -1
    idf, twf = ids.cuda().reshape(-1), d["tw"].cuda().reshape(-1)
    lib, stream = L.load(), torch.cuda.current_stream().cuda_stream
    numel = T * topk
    c2 = torch.full((numel, inter), 7.0, dtype=torch.bfloat16, device="cuda")
    xd = d["x"].cuda()
    L.check(lib.ksq_moe_w4a16_gate_up_silu(c2.data_ptr(), xd.data_ptr(), w13p.data_ptr(), s13p.data_ptr(), None,
                                           None, idf.data_ptr(), None, numel, topk, E, 2 * inter, hidden, 128, 16, H.BF16, stream))
    assert torch.all(c2[1] == 7.0) and torch.all(c2[6] == 7.0)          # untouched rows
    out = torch.empty((T, hidden), dtype=torch.bfloat16, device="cuda")
    L.check(lib.ksq_moe_w4a16_down_sum(out.data_ptr(), c2.data_ptr(), w2p.data_ptr(), s2p.data_ptr(), twf.data_ptr(),
                                       idf.data_ptr(), T, topk, E, hidden, inter, 128, H.BF16, stream))
    # the same with the two slots routed to a real expert at weight zero
    ids2, tw2 = ids.clone(), d["tw"].clone()
    ids2[0, 1], ids2[1, 2] = 0, 0
    tw2[0, 1], tw2[1, 2] = 0.0, 0.0
    out2 = torch.empty_like(out)
    c2b = c2.clone()
    c2b[1], c2b[6] = 0, 0
    tw2f, ids2f = tw2.cuda().reshape(-1), ids2.cuda().reshape(-1)
    L.check(lib.ksq_moe_w4a16_down_sum(out2.data_ptr(), c2b.data_ptr(), w2p.data_ptr(), s2p.data_ptr(), tw2f.data_ptr(),
                                       ids2f.data_ptr(), T, topk, E, hidden, inter, 128, H.BF16, stream))
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    assert lib.ksq_moe_w4a16_down_sum(out.data_ptr(), c2.data_ptr(), w2p.data_ptr(), s2p.data_ptr(), twf.data_ptr(),
                                      idf.data_ptr(), 9, topk, E, hidden, inter, 128, H.BF16, stream) == 1
    assert lib.ksq_moe_w4a16_gemm(out.data_ptr(), c2.data_ptr(), w2p.data_ptr(), s2p.data_ptr(), None, None, None,
                                  idf.data_ptr(), None, numel, 1, E, hidden, inter, 128, 32, H.BF16, stream) == 1


# ---- block-quantized fp8 experts -------------------------------------------------------------------------------------

def _fp8_experts(oracle, seed, E, n, k):
    g = H.gen(seed)
    w = (torch.randn((E, n, k), generator=g) * 0.02).to(torch.bfloat16).float().numpy()
    q = np.empty((E, n, k), np.uint8)
    s = np.empty((E, (n + 127) // 128, k // 128), np.float32)
    for e in range(E):
        q[e], s[e] = oracle.fp8_block_quant_weight(w[e])
    return q, s


@pytest.mark.parametrize("T,E,topk,n,k,bm,colmajor,with_w", [
    (1, 8, 2, 256, 256, 16, False, False), (70, 8, 2, 208, 384, 16, True, True), (300, 6, 3, 512, 1024, 32, False, True),
    (33, 16, 4, 4096, 7168, 32, False, False),
    # 256-slot blocks: the MFMA tile kernel in its grouped form (ragged n, both scale layouts, routing weight)
    (300, 6, 3, 512, 1024, 256, False, True), (700, 4, 2, 784, 512, 256, True, False), (130, 2, 1, 256, 128, 256, False, True),
    # 128-slot blocks of the same kernel
    (300, 6, 3, 512, 1024, 128, False, True), (700, 4, 2, 784, 512, 128, True, False), (130, 2, 1, 256, 128, 128, False, True),
    (90, 3, 2, 2064, 640, 128, True, True)])
def test_grouped_fp8_gemm_stage(ops, oracle, T, E, topk, n, k, bm, colmajor, with_w):
    """One grouped blockwise-fp8 GEMM launch against the per-expert oracle GEMM on the codes the GPU quantizer wrote."""
    g = H.gen(7000 + T + n)
    bq, bs = _fp8_experts(oracle, 7100 + n, E, n, k)
    x = torch.randn((T, k), generator=g).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(T)]).to(torch.int32)
    tw = torch.rand((T, topk), generator=g)
    numel = T * topk
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, colmajor)
    sorted_ids, expert_ids, npp = ops.moe_align_block_size(ids.cuda(), E, bm)
    out = ops.moe_fp8_blockwise_gemm(q, s, colmajor, ops.fp8_repack_weight(torch.from_numpy(bq).cuda()), torch.from_numpy(bs).cuda(),
                                     tw.reshape(-1).cuda() if with_w else None, sorted_ids, expert_ids, npp, numel, topk,
                                     bm, torch.bfloat16)
    qh, sh = q.cpu().numpy(), s.cpu().numpy()
    ref = np.zeros((numel, n), np.float32)
    flat = ids.reshape(-1).numpy()
    for e in range(E):
        slots = np.nonzero(flat == e)[0]
        if slots.size:
            rows = slots // topk
            a_s = sh[:, rows] if colmajor else sh[rows]
            ref[slots] = oracle.fp8_blockwise_gemm(qh[rows], np.ascontiguousarray(a_s), bq[e], bs[e], colmajor)
    if with_w:
        ref *= tw.reshape(-1, 1).numpy()
    H.check_gemm(out, ref, H.BF16, "grouped fp8 T=%d n=%d k=%d" % (T, n, k))


@pytest.mark.parametrize("bm", [128, 256])
def test_grouped_fp8_tile_kernel_every_count_of_live_row_tiles(ops, oracle, bm):
    """Every wavefront of the fp8 tile kernel has an instance of its main loop per number of its row tiles that hold
    tokens: experts with 16c - 5 slots for c = 1..16 meet every count of the lower and of the upper wavefronts of a
    256-slot block (cut into 128-slot blocks: of that form)."""
    rows = [16 * c - 5 for c in range(1, 17)]
    E, T, n, k = len(rows), sum(rows), 256, 384
    g = H.gen(7700 + bm)
    bq, bs = _fp8_experts(oracle, 7710, E, n, k)
    x = torch.randn((T, k), generator=g).to(torch.bfloat16)
    ids = torch.cat([torch.full((r,), e, dtype=torch.int32) for e, r in enumerate(rows)])
    ids = ids[torch.randperm(T, generator=g)].reshape(T, 1).contiguous()
    q, s = ops.per_token_group_quant_fp8(x.cuda(), k, 128, False)
    sorted_ids, expert_ids, npp = ops.moe_align_block_size(ids.cuda(), E, bm)
    out = ops.moe_fp8_blockwise_gemm(q, s, False, ops.fp8_repack_weight(torch.from_numpy(bq).cuda()), torch.from_numpy(bs).cuda(),
                                     None, sorted_ids, expert_ids, npp, T, 1, bm, torch.bfloat16)
    qh, sh = q.cpu().numpy(), s.cpu().numpy()
    ref = np.zeros((T, n), np.float32)
    flat = ids.reshape(-1).numpy()
    for e in range(E):
        slots = np.nonzero(flat == e)[0]
        ref[slots] = oracle.fp8_blockwise_gemm(qh[slots], np.ascontiguousarray(sh[slots]), bq[e], bs[e], False)
    H.check_gemm(out, ref, H.BF16, "grouped fp8 tile kernel, %d-slot blocks" % bm)


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("T,E,topk,hidden,inter", [(1, 8, 2, 256, 128), (48, 16, 4, 512, 256), (200, 8, 2, 384, 640),
                                                   (1200, 8, 2, 512, 256)])   # the last: 300 slots per expert, 256-slot blocks
def test_moe_fp8_block(ops, oracle, dtype, T, E, topk, hidden, inter):
    """Whole block-fp8 MoE block.  The silu*mul front end of the second quantization rounds through T once more than
    the oracle may (see the quantizer's fused test), so the block is compared at GEMM tolerance, not bit for bit."""
    g = H.gen(7300 + T + hidden)
    w13, s13 = _fp8_experts(oracle, 7400 + hidden, E, 2 * inter, hidden)
    w2, s2 = _fp8_experts(oracle, 7500 + hidden, E, hidden, inter)
    x = torch.randn((T, hidden), generator=g).to(H.TORCH_DT[dtype])
    logits = torch.randn((T, E), generator=g)
    tw, ids = ops.moe_topk_softmax(logits.cuda(), topk, True, 1.0)
    y = ops.fused_moe_fp8_blockwise(x.cuda(), ops.fp8_repack_weight(torch.from_numpy(w13).cuda()), torch.from_numpy(s13).cuda(),
                                    ops.fp8_repack_weight(torch.from_numpy(w2).cuda()), torch.from_numpy(s2).cuda(), ids, tw)
    ref = oracle.moe_fp8_forward(H.bits_of(x), w13, s13, w2, s2, ids.cpu().numpy(), tw.cpu().numpy(), dtype)
    H.check_gemm(y, oracle.from_bits(ref, dtype), dtype, "fp8 moe block")


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("T,E,topk,hidden,inter", [(1, 8, 2, 256, 128), (2, 16, 8, 512, 256), (4, 8, 4, 384, 640), (8, 8, 2, 256, 384)])
def test_few_tokens_fp8_without_alignment_and_with_the_sum_in_the_second_gemm(ops, oracle, dtype, T, E, topk, hidden, inter):
    """Block-fp8 experts, a handful of slots: the first GEMM with every slot a block of its own gives the bits of the
    aligned form; the second GEMM with the sum over top-k in it is held against the fp32 sum of the oracle's rows for
    the very codes and scales it read."""
    from ksanallm_amd import lib as L
    g = H.gen(7600 + T + hidden)
    w13, s13 = _fp8_experts(oracle, 7700 + hidden, E, 2 * inter, hidden)
    w2, s2 = _fp8_experts(oracle, 7800 + hidden, E, hidden, inter)
    w13p, s13d = ops.fp8_repack_weight(torch.from_numpy(w13).cuda()), torch.from_numpy(s13).cuda()
    w2p, s2d = ops.fp8_repack_weight(torch.from_numpy(w2).cuda()), torch.from_numpy(s2).cuda()
    td = H.TORCH_DT[dtype]
    x = torch.randn((T, hidden), generator=g).to(td).cuda()
    tw, ids = ops.moe_topk_softmax(torch.randn((T, E), generator=g).cuda(), topk, True, 1.0)
    numel = T * topk
    idf, twf = ids.reshape(-1).contiguous(), tw.reshape(-1).contiguous()
    a1_q, a1_s = ops.per_token_group_quant_fp8(x, hidden, 128, False)
    s, e, npp = ops.moe_align_block_size(ids, E, 16)
    want1 = ops.moe_fp8_blockwise_gemm(a1_q, a1_s, False, w13p, s13d, None, s, e, npp, numel, topk, 16, td)
    c1 = ops.moe_fp8_blockwise_gemm(a1_q, a1_s, False, w13p, s13d, None, None, idf, None, numel, topk, 16, td)
    assert torch.equal(c1.view(torch.int16), want1.view(torch.int16))
    a2_q, a2_s = ops.per_token_group_quant_fp8(c1, inter, 128, False, fuse_silu_mul=True)
    want3 = ops.moe_fp8_blockwise_gemm(a2_q, a2_s, False, w2p, s2d, twf, s, e, npp, numel, 1, 16, td)
    c3 = ops.moe_fp8_blockwise_gemm(a2_q, a2_s, False, w2p, s2d, twf, None, idf, None, numel, 1, 16, td)
    assert torch.equal(c3.view(torch.int16), want3.view(torch.int16))
    out = torch.full((T, hidden), float("nan"), dtype=td, device="cuda")
    L.check(L.load().ksq_moe_fp8_down_sum(out.data_ptr(), a2_q.data_ptr(), a2_s.data_ptr(), w2p.data_ptr(), s2d.data_ptr(),
                                          twf.data_ptr(), idf.data_ptr(), T, topk, E, hidden, inter, dtype,
                                          torch.cuda.current_stream().cuda_stream))
    aq, asc, flat, twn = a2_q.cpu().numpy(), a2_s.cpu().numpy(), idf.cpu().numpy(), twf.cpu().numpy()
    rows = np.zeros((numel, hidden), np.float64)
    for slot in range(numel):
        rows[slot] = oracle.fp8_blockwise_gemm(aq[slot:slot + 1], asc[slot:slot + 1], w2[flat[slot]], s2[flat[slot]], False)[0] * twn[slot]
    H.check_gemm(out, rows.reshape(T, topk, hidden).sum(1).astype(np.float32), dtype, "fp8 down + sum T=%d" % T)
    if T <= ops.FEW_TOKENS:
        whole = ops.fused_moe_fp8_blockwise(x, w13p, s13d, w2p, s2d, ids, tw)
        assert torch.equal(whole.view(torch.int16), out.view(torch.int16))
        ref = oracle.moe_fp8_forward(H.bits_of(x.cpu()), w13, s13, w2, s2, ids.cpu().numpy(), tw.cpu().numpy(), dtype)
        # the reference's sequence rounds every expert's share to T and adds them in T; this form keeps fp32 to the end
        # and is held to the bar above - against the reference's own rounding it may differ by that rounding
        H.check_gemm(whole, oracle.from_bits(ref, dtype), dtype, "fp8 few-token block", weights_rounded=True,
                     rel_l2_max=5e-3 + 2.0 ** (-8 if dtype == H.BF16 else -11) * topk ** 0.5)


# ---- full-size properties (DeepSeek-V3 expert shapes: 256 experts, hidden 7168, inter 2048, top-8), no oracle needed:
# a token's output depends on its own row, its experts and its routing weights only, so a permutation of the tokens
# permutes the outputs bit for bit (whatever blocks, tiles and kernels the sizes select), a token routed with zero
# weights comes out as exact zeros, and the same token repeated gives the same row every time.
def _full_size_experts(ops, kind, distinct=16):
    from ksanallm_amd import lib as L
    E, hidden, inter = 256, 7168, 2048
    g = H.gen(9900)
    rep = E // distinct
    if kind == "int4":
        w13 = torch.randint(0, 256, (distinct, 2 * inter, hidden // 2), generator=g, dtype=torch.uint8)
        w2 = torch.randint(0, 256, (distinct, hidden, inter // 2), generator=g, dtype=torch.uint8)
        s13 = H.uniform(g, (distinct, 2 * inter, hidden // 128), 0.002, 0.01, H.BF16)
        s2 = H.uniform(g, (distinct, hidden, inter // 128), 0.002, 0.01, H.BF16)
        return (ops.repack_weight(w13.cuda(), L.SRC_MOE_NK, distinct, hidden, 2 * inter).repeat(rep),
                ops.repack_scales(s13.cuda(), L.SCALE_NG, distinct, hidden, 2 * inter, 128).repeat(rep),
                ops.repack_weight(w2.cuda(), L.SRC_MOE_NK, distinct, inter, hidden).repeat(rep),
                ops.repack_scales(s2.cuda(), L.SCALE_NG, distinct, inter, hidden, 128).repeat(rep))

    def experts(n, k):
        q = torch.randint(0, 256, (distinct, n, k), generator=g, dtype=torch.uint8)
        q = torch.where((q & 0x7f) == 0x7f, q & 0xfe, q)     # no NaN codes
        s = torch.rand((distinct, n // 128, k // 128), generator=g) * 1e-4 + 1e-4
        return ops.fp8_repack_weight(q.cuda()).repeat(rep, 1, 1), s.cuda().repeat(rep, 1, 1)

    w13, s13 = experts(2 * inter, hidden)
    w2, s2 = experts(hidden, inter)
    return w13, s13, w2, s2


@pytest.mark.parametrize("kind", ["int4", "fp8"])
@pytest.mark.parametrize("T", [24, 512, 700, 2304, 4096])      # 16-row, 32-row and tile-kernel blocks; 512 and 4096 are benchmark sizes
def test_moe_full_size_properties(ops, kind, T):
    E, hidden, inter, topk = 256, 7168, 2048, 8
    w13, s13, w2, s2 = _full_size_experts(ops, kind)
    g = H.gen(9950 + T)
    x = torch.randn((T, hidden), generator=g).to(torch.bfloat16)
    x[T // 2] = x[0]                                    # a repeated token
    logits = torch.randn((T, E), generator=g)
    logits[T // 2] = logits[0]
    tw, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
    tw = tw.float().contiguous()
    tw[1] = 0.0                                         # a token whose routing weights are all zero
    ids = ids.to(torch.int32)

    def run(xx, ii, ww):
        if kind == "int4":
            return ops.fused_moe_w4a16(xx.cuda(), w13, s13, w2, s2, ii.cuda(), ww.cuda(), E, hidden, inter, 128)
        return ops.fused_moe_fp8_blockwise(xx.cuda(), w13, s13, w2, s2, ii.cuda(), ww.cuda())

    y = run(x, ids, tw)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    assert torch.count_nonzero(y[1]) == 0
    assert torch.equal(y[0].view(torch.int16), y[T // 2].view(torch.int16))
    perm = torch.randperm(T, generator=g)
    yp = run(x[perm], ids[perm], tw[perm])
    torch.cuda.synchronize()
    assert torch.equal(yp.view(torch.int16), y[perm.cuda()].view(torch.int16))


@pytest.mark.parametrize("dtype", [H.F16, H.BF16])
@pytest.mark.parametrize("tokens,top_k,E,k", [(1, 4, 8, 128), (37, 2, 16, 384), (300, 8, 64, 2048),
                                               (200, 2, 4, 36), (130, 2, 2, 40960)])   # the last two: rows the LDS form does not take
def test_moe_permute_columns_bit_exact(ops, dtype, tokens, top_k, E, k):
    """out[s, j] = x[s // top_k, perm[ids[s], j]] for the first MoE GEMM, and with top_k = 1 (one input row per slot)
    for the second."""
    g = H.gen(tokens + k)
    x = torch.randn((tokens, k), generator=g).to(H.TORCH_DT[dtype])
    perm = torch.stack([torch.randperm(k, generator=g) for _ in range(E)]).to(torch.int32)
    ids = torch.randint(0, E, (tokens * top_k,), generator=g, dtype=torch.int32)
    out = ops.moe_permute_columns(x.cuda(), perm.cuda(), ids.cuda(), top_k)
    rows = torch.arange(tokens * top_k) // top_k
    ref = torch.gather(x[rows], 1, perm[ids.long()].long())
    assert torch.equal(out.cpu(), ref)
    xs = torch.randn((tokens * top_k, k), generator=g).to(H.TORCH_DT[dtype])
    out1 = ops.moe_permute_columns(xs.cuda(), perm.cuda(), ids.cuda(), 1)
    assert torch.equal(out1.cpu(), torch.gather(xs, 1, perm[ids.long()].long()))


@pytest.mark.parametrize("m,k", [(1, 128), (50, 7168), (300, 2048), (1000, 7168), (300, 36), (260, 40960)])
def test_permute_columns_bit_exact(ops, m, k):
    """out[r, j] = x[r, perm[j]]: rows staged in LDS (from 256 rows, k a multiple of 8 and at most 32768) and the direct
    form."""
    g = H.gen(m + k)
    x = torch.randn((m, k), generator=g).to(torch.bfloat16)
    perm = torch.randperm(k, generator=g).to(torch.int32)
    out = ops.permute_columns(x.cuda(), perm.cuda())
    assert torch.equal(out.cpu(), x[:, perm.long()])
