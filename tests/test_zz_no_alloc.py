"""ksq_w4a16_gemm_static: the W4A16 GEMM whose scratch is a buffer inside the library, against ksq_w4a16_gemm with a
caller's workspace - the same kernels on the same plan, so the outputs must agree bit for bit.  Two calls in a row, the
second on a smaller problem, both with plans that use the scratch (fp32 partial sums of launches that cut K)."""
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


def _problem(ops, L, seed, M, N, K, dtype, awq, group=128):
    d = H.make_w4a16(seed, M, N, K, group, dtype, awq=awq, x_std=0.5, s_lo=0.002, s_hi=0.01, z_lo=0, z_hi=15)
    wp = ops.repack_weight(d["qweight"].cuda(), L.SRC_AWQ if awq else L.SRC_GPTQ, 1, K, N)
    sp = ops.repack_scales(d["scales"].cuda(), L.SCALE_GN, 1, K, N, group)
    zp = ops.repack_zeros(d["qzeros"].cuda(), L.ZERO_AWQ_PACKED, K, N, group) if awq else None
    return d, d["x"].cuda(), wp, sp, zp


def _static(L, x, wp, sp, zp, N, K, dtype, group=128, y=None):
    if y is None:
        y = torch.full((x.shape[0], N), float("nan"), dtype=x.dtype, device=x.device)
    L.check(L.load().ksq_w4a16_gemm_static(y.data_ptr(), x.data_ptr(), wp.data_ptr(), sp.data_ptr(),
                                           None if zp is None else zp.data_ptr(), x.shape[0], N, K, group, dtype,
                                           torch.cuda.current_stream().cuda_stream))
    return y


@pytest.mark.parametrize("small_problem_rule", [True, False])
@pytest.mark.parametrize("dtype,awq", [(H.BF16, True), (H.F16, False)])
def test_static_scratch_matches_workspace_form(dtype, awq, small_problem_rule):
    from ksanallm_amd import lib as L
    from ksanallm_amd import ops
    lib = L.load()
    L.set_small_problem_rule(small_problem_rule)  # off: the two problems of more than 32 rows run the tile kernel
    cap = lib.ksq_w4a16_static_workspace_bytes()
    assert cap == 32 << 20
    # a problem of 128 rows with K cut over workgroups (decode form over four row blocks, or the tile kernel), then the
    # decode kernel with K cut over workgroups on a smaller problem, then a plan that needs no scratch at all
    shapes = [(128, 4096, 14336), (8, 1024, 4096), (64, 512, 2048), (3, 768, 256)]
    for i, (M, N, K) in enumerate(shapes):
        need = lib.ksq_w4a16_workspace_size(M, N, K, 128, dtype)
        assert need <= cap and (need > 0 or i == 3), (M, N, K, need)
        d, x, wp, sp, zp = _problem(ops, L, 8100 + i, M, N, K, dtype, awq)
        ref = ops.w4a16_gemm(x, wp, sp, zp, N, K, 128)
        y = _static(L, x, wp, sp, zp, N, K, dtype)
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), ref.view(torch.int16)), (M, N, K)
        H.check_gemm(y, H.w4a16_oracle(d), dtype, "static scratch M=%d N=%d K=%d" % (M, N, K), weights_rounded=M > 32)
    # the first problem once more: what the smaller calls left in the buffer must not show
    M, N, K = shapes[0]
    d, x, wp, sp, zp = _problem(ops, L, 8100, M, N, K, dtype, awq)
    assert torch.equal(_static(L, x, wp, sp, zp, N, K, dtype).view(torch.int16),
                       ops.w4a16_gemm(x, wp, sp, zp, N, K, 128).view(torch.int16))


def test_static_scratch_rejects_plans_beyond_its_size(tile_kernels):
    from ksanallm_amd import lib as L
    lib = L.load()
    cap = lib.ksq_w4a16_static_workspace_bytes()
    # a shape whose plan for this very m needs more than the buffer holds
    found = None
    for (M, N, K) in [(256, 8192, 28672), (200, 16384, 16384), (256, 14336, 8192), (256, 25600, 5120), (150, 12288, 12288)]:
        d1 = L.select_tile(L.KIND_W4A16, M, N, K, H.BF16)
        if d1["kernel"] == 1 and d1["split_k"] > 1 and lib.ksq_w4a16_workspace_size(M, N, K, 128, H.BF16) > cap:
            # the workspace query is a maximum over all m up to M; the entry point looks at M alone
            found = (M, N, K)
            break
    if found is None:
        pytest.skip("no probe shape needs more scratch than the buffer holds")
    M, N, K = found
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(K * N // 2, dtype=torch.uint8, device="cuda")
    s = torch.zeros((K // 128) * N, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    rc = lib.ksq_w4a16_gemm_static(y.data_ptr(), x.data_ptr(), w.data_ptr(), s.data_ptr(), None, M, N, K, 128, H.BF16,
                                   torch.cuda.current_stream().cuda_stream)
    if rc == 0:
        pytest.skip("the plan for m=%d alone fits" % M)
    assert rc == 3 and b"scratch" in lib.ksq_last_error_string()


def test_static_scratch_allocates_nothing_and_replays_from_a_graph(tile_kernels):
    """What the entry point promises beyond its results: the device's free memory is the same after a run of calls as
    before the first of them, and a call captured into a HIP graph (after one eager call on the device, which
    resolves the buffer's address and the kernels' attributes) replays to the eager bits every time, with eager work
    between the replays.  The plans cut K (tile kernel, group 128 and group 64; decode kernel), so the scratch is in
    use."""
    from ksanallm_amd import lib as L
    from ksanallm_amd import ops
    lib = L.load()
    cases = []
    for i, (M, N, K, group) in enumerate([(128, 4096, 14336, 128), (96, 2048, 8192, 64), (8, 1024, 4096, 128)]):
        assert 0 < lib.ksq_w4a16_workspace_size(M, N, K, group, H.BF16) <= lib.ksq_w4a16_static_workspace_bytes()
        d, x, wp, sp, zp = _problem(ops, L, 8200 + i, M, N, K, H.BF16, False, group)
        ref = ops.w4a16_gemm(x, wp, sp, zp, N, K, group)
        H.check_gemm(ref, H.w4a16_oracle(d), H.BF16, "M=%d N=%d K=%d group %d" % (M, N, K, group), weights_rounded=M > 32)
        y = torch.empty_like(ref)
        cases.append((x, wp, sp, zp, N, K, group, ref, y))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        for (x, wp, sp, zp, N, K, group, ref, y) in cases:
            _static(L, x, wp, sp, zp, N, K, H.BF16, group, y)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    for (x, wp, sp, zp, N, K, group, ref, y) in cases:
        assert torch.equal(y.view(torch.int16), ref.view(torch.int16))
    # graph: the three calls in one captured sequence
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for (x, wp, sp, zp, N, K, group, ref, y) in cases:
            y.zero_()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for (x, wp, sp, zp, N, K, group, ref, y) in cases:
                _static(L, x, wp, sp, zp, N, K, H.BF16, group, y)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        for (x, wp, sp, zp, N, K, group, ref, y) in cases:
            y.fill_(float("nan"))
        # eager work that uses the same scratch between the replays
        x, wp, sp, zp, N, K, group, ref, _ = cases[rep % len(cases)]
        assert torch.equal(_static(L, x, wp, sp, zp, N, K, H.BF16, group).view(torch.int16), ref.view(torch.int16))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for (x, wp, sp, zp, N, K, group, ref, y) in cases:
            assert torch.equal(y.view(torch.int16), ref.view(torch.int16)), rep
