"""Pins the W4A8 functions of the CPU oracle (nothing here needs a GPU)."""
import numpy as np
import torch


def test_int4_nibble_split_known_answers(oracle):
    """The reference test's unpack (finegrained_mixed_dtype_gemm_thop_test.cu:53-80): element 0 = the low nibble,
    element 1 = the high nibble, both sign-extended.  Answers written out by hand."""
    w = np.array([[0x8F, 0x70, 0x00, 0xF8, 0x17, 0xE2]], dtype=np.uint8).view(np.int8)
    out = oracle.w4a8_unpack_int4(w)
    np.testing.assert_array_equal(out, np.int8([[-1, -8, 0, 7, 0, 0, -8, -1, 7, 1, 2, -2]]))
    # every byte value: (b << 4) >> 4 and b >> 4 in int8 arithmetic
    allb = np.arange(256, dtype=np.uint8).reshape(1, 256).view(np.int8)
    got = oracle.w4a8_unpack_int4(allb).reshape(256, 2).astype(np.int32)
    b = np.arange(256)
    lo = ((b & 15) ^ 8) - 8
    hi = ((b >> 4) ^ 8) - 8
    np.testing.assert_array_equal(got[:, 0], lo)
    np.testing.assert_array_equal(got[:, 1], hi)


def test_int4_codes_read_as_e4m3_are_multiples_of_2_pow_minus_9(oracle):
    """What the kernel's weight conversion rests on: the byte u (0..15) decodes to u * 2^-9 in OCP e4m3 (the decoder
    itself is checked against torch's float8_e4m3fn in tests/test_oracle_golden.py)."""
    u = np.arange(16, dtype=np.uint8)
    np.testing.assert_array_equal(oracle.e4m3_to_f32(u), u.astype(np.float32) * np.float32(2.0 ** -9))
    np.testing.assert_array_equal(torch.from_numpy(u).view(torch.float8_e4m3fn).float().numpy(),
                                  u.astype(np.float32) * np.float32(2.0 ** -9))


def test_static_quant_matches_torch_cast_of_the_fp32_quotient(oracle):
    rng = np.random.default_rng(11)
    m, k = 6, 256
    x = (rng.standard_normal((m, k)) * rng.choice([1e-3, 0.1, 1, 30, 3000], (m, k))).astype(np.float32)
    for dtype in (0, 1):
        xb = oracle.to_bits(x, dtype)
        xr = oracle.from_bits(xb, dtype)
        for per_channel in (False, True):
            s = (rng.random(k if per_channel else 1) * 2 + 0.01).astype(np.float32)
            q = oracle.w4a8_static_quant(xb, s, per_channel, dtype)
            r = np.clip(xr / (s[None, :] if per_channel else s[0]), -448, 448).astype(np.float32)
            ref = torch.from_numpy(r).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
            np.testing.assert_array_equal(q, ref)
        s = (rng.random(m) * 2 + 0.01).astype(np.float32)
        q = oracle.w4a8_static_quant(xb, s, False, dtype, per_token=True)
        r = np.clip(xr / s[:, None], -448, 448).astype(np.float32)
        np.testing.assert_array_equal(q, torch.from_numpy(r).to(torch.float8_e4m3fn).view(torch.uint8).numpy())
    # saturation and specials
    xs = np.float32([[1e6, -1e6, np.inf, -np.inf, 448, -449, 0.0, -0.0] * 16])
    q = oracle.w4a8_static_quant(oracle.to_bits(xs, 1), np.float32([1.0]), False, 1)
    np.testing.assert_array_equal(q[0, :8], np.uint8([0x7E, 0xFE, 0x7E, 0xFE, 0x7E, 0xFE, 0x00, 0x80]))


def test_group_sums_against_numpy(oracle):
    rng = np.random.default_rng(12)
    q = rng.integers(0, 256, (5, 384), dtype=np.uint8)
    q[(q & 0x7F) == 0x7F] = 0  # no NaN codes
    got = oracle.w4a8_group_sums(q)
    ref = oracle.e4m3_to_f32(q).astype(np.float64).reshape(5, 3, 128).sum(-1)
    np.testing.assert_array_equal(got, ref.astype(np.float32))
    # every e4m3 value is a multiple of 2^-9, so sums of 128 of them below 2^15 are exact in fp32
    assert np.all(ref == got.astype(np.float64))


def test_group_sums_and_gemm_with_group_64(oracle):
    """Group size 64: sums against numpy float64, and the GEMM against the reference test's formula with the scales
    repeated 64 times; scales that are equal in both halves of every 128 give the group-128 result."""
    rng = np.random.default_rng(14)
    m, n, k = 6, 32, 384
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x28
    got = oracle.w4a8_group_sums(a, 64)
    ref = oracle.e4m3_to_f32(a).astype(np.float64).reshape(m, k // 64, 64).sum(-1)
    np.testing.assert_array_equal(got, ref.astype(np.float32))
    w = rng.integers(0, 256, (k, n // 2), dtype=np.uint8).view(np.int8)
    s64 = (rng.random((k // 64, n)) * 0.02 + 0.001).astype(np.float16)
    out = oracle.w4a8_gemm(a, w, s64.view(np.uint16), 0.5, group=64)
    wt = torch.from_numpy(oracle.w4a8_unpack_int4(w)).double()
    sc = torch.from_numpy(s64.astype(np.float64)).repeat_interleave(64, 0)
    act = torch.from_numpy(a).view(torch.float8_e4m3fn).double() * 0.5
    np.testing.assert_allclose(out, (act @ (wt * sc)).numpy(), rtol=2e-7, atol=1e-12)
    s128 = s64[0::2].copy()
    same = np.repeat(s128, 2, axis=0)
    np.testing.assert_array_equal(oracle.w4a8_gemm(a, w, same.view(np.uint16), 0.5, group=64),
                                  oracle.w4a8_gemm(a, w, s128.view(np.uint16), 0.5, group=128))


def test_gemm_is_the_reference_tests_formula(oracle):
    """finegrained_mixed_dtype_gemm_thop_test.cu:186-206 in torch float64: unpack, times the repeated scales, matmul
    with the alpha-scaled activations."""
    rng = np.random.default_rng(13)
    m, n, k = 7, 48, 256
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    a[(a & 0x7F) == 0x7F] = 0x30
    w = rng.integers(0, 256, (k, n // 2), dtype=np.uint8).view(np.int8)
    scales = (rng.random((k // 128, n)) * 0.02 + 0.001).astype(np.float16)
    alpha = 0.37
    got = oracle.w4a8_gemm(a, w, scales.view(np.uint16), alpha)
    wt = torch.from_numpy(oracle.w4a8_unpack_int4(w)).double()
    sc = torch.from_numpy(scales.astype(np.float64)).repeat_interleave(128, 0)
    act = torch.from_numpy(a).view(torch.float8_e4m3fn).double() * float(np.float32(alpha))
    ref = (act @ (wt * sc)).numpy()
    np.testing.assert_allclose(got, ref, rtol=2e-7, atol=1e-12)
    # linear in alpha, and a one-hot activation row reads out one weight row times its scales
    got2 = oracle.w4a8_gemm(a, w, scales.view(np.uint16), 2 * alpha)
    np.testing.assert_allclose(got2, 2 * got, rtol=2e-7)
    onehot = np.zeros((1, k), np.uint8)
    onehot[0, 130] = 0x38  # 1.0
    row = oracle.w4a8_gemm(onehot, w, scales.view(np.uint16), 1.0)[0]
    np.testing.assert_array_equal(row, (oracle.w4a8_unpack_int4(w)[130].astype(np.float32) *
                                        scales[1].astype(np.float32)))


def test_packed_layout_against_a_scalar_loop(oracle):
    """The numpy statement of the packed layout against element-by-element placement on a small weight."""
    rng = np.random.default_rng(14)
    K, N = 256, 32
    w = rng.integers(0, 256, (K, N // 2), dtype=np.uint8).view(np.int8)
    words = oracle.w4a8_repack_weight(w)
    vals = oracle.w4a8_unpack_int4(w).astype(np.int32)
    ref = np.zeros(K * N // 8, np.uint32)
    KB = K // 128
    for k in range(K):
        for n in range(N):
            kb, r = divmod(k, 128)
            q, rr = divmod(r, 32)
            i, e = divmod(rr, 8)
            lane = 16 * q + n % 16
            pos = 2 * e if e < 4 else 2 * (e - 4) + 1
            word = ((n // 16) * KB + kb) * 256 + lane * 4 + i
            ref[word] |= np.uint32((vals[k, n] + 8) << (4 * pos))
    np.testing.assert_array_equal(words, ref)
