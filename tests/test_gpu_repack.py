"""Load-time repack: bit-exact round trip through the CDNA4 tile layout for every checkpoint layout, and the layout
itself checked against an index-level restatement in numpy."""
import numpy as np
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


def packed_reference(codes):
    """codes [E, K, N] u8 -> packed dwords as documented in include/ksq.h (numpy restatement of the layout)."""
    E, K, N = codes.shape
    c = codes.reshape(E, K // 128, 4, 4, 8, N // 16, 16)  # e, kt, d, kq, j, nt, nn
    c = c.transpose(0, 5, 1, 3, 6, 2, 4)                  # e, nt, kt, kq, nn, d, j  (lane = kq*16+nn)
    order = [0, 2, 4, 6, 1, 3, 5, 7]                      # nibble p holds j = order[p]
    w = np.zeros(c.shape[:-1], dtype=np.uint32)
    for p, j in enumerate(order):
        w |= c[..., j].astype(np.uint32) << np.uint32(4 * p)
    return w.reshape(-1)


@pytest.fixture(scope="module")
def ops():
    from ksanallm_amd import ops
    return ops


@pytest.mark.parametrize("K,N", [(128, 16), (256, 48), (4096, 4096)])
def test_gptq_awq_int4x2_roundtrip(ops, oracle, K, N):
    from ksanallm_amd import lib as L
    rng = np.random.default_rng(K + N)
    codes = rng.integers(0, 16, (K, N), dtype=np.uint8)
    ref = packed_reference(codes[None])
    srcs = {
        L.SRC_GPTQ: oracle.gptq_pack(codes).view(np.int32),
        L.SRC_AWQ: oracle.awq_pack(codes).view(np.int32),
        L.SRC_INT4X2_KN: oracle.pack_int8_to_int4x2((codes.astype(np.int16) - 8).astype(np.int8)),
    }
    for layout, src in srcs.items():
        d_src = torch.from_numpy(src).cuda()
        packed = ops.repack_weight(d_src, layout, 1, K, N)
        got = packed.cpu().numpy().view(np.uint32)
        np.testing.assert_array_equal(got, ref, err_msg="layout %d" % layout)
        back = ops.unpack_weight(packed, layout, 1, K, N).cpu().numpy()
        np.testing.assert_array_equal(back, src, err_msg="layout %d" % layout)


def test_every_nibble_position_and_value(ops, oracle):
    """Exhaustive over the 1024 positions of a tile x 16 code values: a single non-zero code must come back alone."""
    from ksanallm_amd import lib as L
    K, N = 128, 16
    base = np.zeros((K, N), np.uint8)
    srcs = []
    for k in range(0, K, 7):
        for n in range(N):
            c = base.copy()
            c[k, n] = (k * 3 + n) % 15 + 1
            srcs.append(c)
    stack = np.stack(srcs)  # [E, K, N] used as E independent matrices
    E = stack.shape[0]
    q = np.stack([oracle.gptq_pack(c) for c in stack]).view(np.int32)
    d = torch.from_numpy(q).cuda()
    packed = ops.repack_weight(d, L.SRC_GPTQ, E, K, N)
    np.testing.assert_array_equal(packed.cpu().numpy().view(np.uint32), packed_reference(stack))
    back = ops.unpack_weight(packed, L.SRC_GPTQ, E, K, N).cpu().numpy()
    np.testing.assert_array_equal(back, q)


def test_moe_layout_roundtrip(ops, oracle):
    from ksanallm_amd import lib as L
    rng = np.random.default_rng(5)
    E, K, N = 6, 256, 64
    codes = rng.integers(0, 16, (E, K, N), dtype=np.uint8)
    w = oracle.moe_pack(codes)  # [E, N, K/2]
    d = torch.from_numpy(w).cuda()
    packed = ops.repack_weight(d, L.SRC_MOE_NK, E, K, N)
    np.testing.assert_array_equal(packed.cpu().numpy().view(np.uint32), packed_reference(codes))
    np.testing.assert_array_equal(ops.unpack_weight(packed, L.SRC_MOE_NK, E, K, N).cpu().numpy(), w)


def test_scales_and_zeros_roundtrip(ops, oracle):
    from ksanallm_amd import lib as L
    g = H.gen(11)
    K, N, group = 512, 96, 128
    for dt in (torch.float16, torch.bfloat16):
        s = torch.rand((K // group, N), generator=g).to(dt)
        ps = ops.repack_scales(s.cuda(), L.SCALE_GN, 1, K, N, group)
        ref = s.view(K // group, N // 16, 16).permute(1, 0, 2).contiguous().view(-1)
        assert torch.equal(ps.cpu(), ref)
        assert torch.equal(ops.unpack_scales(ps, L.SCALE_GN, 1, K, N, group).cpu(), s)
        E = 3
        sm = torch.rand((E, N, K // group), generator=g).to(dt)
        pm = ops.repack_scales(sm.cuda(), L.SCALE_NG, E, K, N, group)
        refm = sm.view(E, N // 16, 16, K // group).permute(0, 1, 3, 2).contiguous().view(-1)
        assert torch.equal(pm.cpu(), refm)
        assert torch.equal(ops.unpack_scales(pm, L.SCALE_NG, E, K, N, group).cpu(), sm)
    z = torch.randint(0, 16, (K // group, N), generator=g, dtype=torch.uint8)
    qz = torch.from_numpy(oracle.awq_pack(z.numpy()).view(np.int32))
    refz = z.view(K // group, N // 16, 16).permute(1, 0, 2).contiguous().view(-1)
    pz = ops.repack_zeros(qz.cuda(), L.ZERO_AWQ_PACKED, K, N, group)
    assert torch.equal(pz.cpu(), refz)
    assert torch.equal(ops.unpack_zeros(pz, L.ZERO_AWQ_PACKED, K, N, group).cpu(), qz)
    pz2 = ops.repack_zeros(z.cuda(), L.ZERO_U8_GN, K, N, group)
    assert torch.equal(pz2.cpu(), refz)
    assert torch.equal(ops.unpack_zeros(pz2, L.ZERO_U8_GN, K, N, group).cpu(), z)


def test_full_size_roundtrip_checksum(ops):
    """Qwen-32B-like weight (K=25600, N=5120): unpack(repack(x)) == x and the multiset of codes is preserved."""
    from ksanallm_amd import lib as L
    K, N = 25600, 5120
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    q = torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, device="cuda", generator=g)
    packed = ops.repack_weight(q, L.SRC_GPTQ, 1, K, N)
    assert torch.equal(ops.unpack_weight(packed, L.SRC_GPTQ, 1, K, N), q)
    def nibble_hist(t):
        b = t.view(torch.uint8).reshape(-1)
        return torch.bincount((b & 15).int(), minlength=16) + torch.bincount((b >> 4).int(), minlength=16)
    assert torch.equal(nibble_hist(packed), nibble_hist(q))


def test_repack_rows_and_gather_columns(ops, oracle):
    """Padded act-order packing: packed row j takes checkpoint row rows[j], index -1 is a padding row with code 8; the
    activation side gathers the same columns and reads 0 for the padding."""
    from ksanallm_amd import lib as L
    K_src, K_dst, N, m = 256, 384, 64, 5
    g = H.gen(77)
    codes = torch.randint(0, 16, (K_src, N), generator=g, dtype=torch.uint8).numpy()
    rows = torch.full((K_dst,), -1, dtype=torch.int32)
    pick = torch.randperm(K_dst, generator=g)[:K_src].sort().values
    rows[pick] = torch.randperm(K_src, generator=g).to(torch.int32)
    q = torch.from_numpy(oracle.gptq_pack(codes).view(np.int32)).cuda()
    dst = torch.empty(K_dst * N // 2, dtype=torch.uint8, device="cuda")
    rows_d = rows.cuda()
    L.check(L.load().ksq_w4a16_repack_rows(q.data_ptr(), rows_d.data_ptr(), dst.data_ptr(), K_src, K_dst, N,
                                           torch.cuda.current_stream().cuda_stream))
    want = np.full((K_dst, N), 8, dtype=np.uint8)
    want[rows.numpy() >= 0] = codes[rows.numpy()[rows.numpy() >= 0]]
    ref = ops.repack_weight(torch.from_numpy(oracle.gptq_pack(want).view(np.int32)).cuda(), L.SRC_GPTQ, 1, K_dst, N)
    assert torch.equal(dst, ref)
    x = torch.randn((m, K_src), generator=g).to(torch.bfloat16)
    out = torch.empty((m, K_dst), dtype=torch.bfloat16, device="cuda")
    x_d = x.cuda()
    L.check(L.load().ksq_gather_columns(x_d.data_ptr(), rows_d.data_ptr(), out.data_ptr(), m, K_src, K_dst, L.BF16,
                                        torch.cuda.current_stream().cuda_stream))
    expect = torch.zeros((m, K_dst), dtype=torch.bfloat16)
    expect[:, rows >= 0] = x[:, rows[rows >= 0].long()]
    assert torch.equal(out.cpu(), expect)
