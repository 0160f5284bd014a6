"""ctypes/numpy front end of the CPU oracle (oracle/ksq_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.  The product package never imports this module.

All arrays are numpy; 16-bit floats travel as ``uint16`` bit patterns so that the oracle
sees exactly the bits the GPU sees.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libksq_oracle.so")

F16, BF16, F32 = 0, 1, 2


def build(force=False):
    """Compile the oracle with gcc (a few seconds)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "ksq_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B"], stdout=subprocess.DEVNULL)
    return _SO


_REF_SO = os.path.join(_HERE, "_ref", "libksq_ref.so")
_REF_HEADER = "/root/reference/3rdparty/LLM_kernels/tests/references/deepseek_v3_grouped_topk.h"


def build_ref():
    """Compile the reference's own host router (oracle/ref_grouped_topk.cpp around its header) into oracle/_ref/ where
    the reference tree is present; returns the library path or None."""
    if os.path.exists(_REF_HEADER):
        subprocess.check_call(["make", "-C", _HERE, "-B", "ref"], stdout=subprocess.DEVNULL)
    return _REF_SO if os.path.exists(_REF_SO) else None


_ref = None


def ref_grouped_topk(gating_f32, bias_f32, top_k, groups, topk_group, scaling):
    """RunDeepSeekV3GroupedTopkRef<float> of the reference (sigmoid scores, bias-corrected choice, top-2 group rank,
    renormalized weights times `scaling`) from oracle/_ref; None when that library has not been built."""
    global _ref
    if _ref is None:
        if not os.path.exists(_REF_SO):
            return None
        _ref = ctypes.CDLL(_REF_SO)
    g = np.ascontiguousarray(gating_f32, np.float32)
    b = np.ascontiguousarray(bias_f32, np.float32)
    T, E = g.shape
    w = np.zeros((T, top_k), np.float32)
    ids = np.zeros((T, top_k), np.int32)
    _ref.ksq_ref_grouped_topk(_p(g), _p(b), ctypes.c_float(scaling), _p(w), _p(ids), ctypes.c_int(T), ctypes.c_int(E),
                              ctypes.c_int(top_k), ctypes.c_int(groups), ctypes.c_int(topk_group))
    return w, ids


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.ksqo_f16_to_f32.restype = ctypes.c_float
        _lib.ksqo_f16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.ksqo_f32_to_f16.restype = ctypes.c_uint16
        _lib.ksqo_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.ksqo_f32_to_e4m3.restype = ctypes.c_uint8
        _lib.ksqo_f32_to_e4m3.argtypes = [ctypes.c_float]
        _lib.ksqo_e4m3_to_f32.restype = ctypes.c_float
        _lib.ksqo_e4m3_to_f32.argtypes = [ctypes.c_uint8]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _sz(v):
    return ctypes.c_size_t(int(v))


# ---------------------------------------------------------------- scalar formats
def _bulk(fn, src, src_dt, dst_dt):
    src = _c(src, src_dt)
    dst = np.empty(src.shape, dtype=dst_dt)
    getattr(lib(), fn)(_p(src), _p(dst), _sz(src.size))
    return dst


def f16_to_f32(h):
    return _bulk("ksqo_f16_to_f32_n", h, np.uint16, np.float32)


def f32_to_f16(f):
    return _bulk("ksqo_f32_to_f16_n", f, np.float32, np.uint16)


def bf16_to_f32(h):
    return _bulk("ksqo_bf16_to_f32_n", h, np.uint16, np.float32)


def f32_to_bf16(f):
    return _bulk("ksqo_f32_to_bf16_n", f, np.float32, np.uint16)


def e4m3_to_f32(c):
    return _bulk("ksqo_e4m3_to_f32_n", c, np.uint8, np.float32)


def f32_to_e4m3(f):
    return _bulk("ksqo_f32_to_e4m3_n", f, np.float32, np.uint8)


def to_bits(f, dtype):
    """float32 array -> storage array of ``dtype`` (uint16 bits for f16/bf16)."""
    if dtype == F16:
        return f32_to_f16(f)
    if dtype == BF16:
        return f32_to_bf16(f)
    return _c(f, np.float32)


def from_bits(b, dtype):
    if dtype == F16:
        return f16_to_f32(b)
    if dtype == BF16:
        return bf16_to_f32(b)
    return _c(b, np.float32)


def _store_dt(dtype):
    return np.float32 if dtype == F32 else np.uint16


# ---------------------------------------------------------------- checkpoint layouts
def gptq_unpack(qweight):
    q = _c(qweight, np.uint32)
    K, N = q.shape[0] * 8, q.shape[1]
    out = np.empty((K, N), np.uint8)
    lib().ksqo_gptq_unpack(_p(q), _p(out), _sz(K), _sz(N))
    return out


def gptq_pack(codes):
    c = _c(codes, np.uint8)
    K, N = c.shape
    out = np.empty((K // 8, N), np.uint32)
    lib().ksqo_gptq_pack(_p(c), _p(out), _sz(K), _sz(N))
    return out


def awq_unpack(q):
    q = _c(q, np.uint32)
    R, N = q.shape[0], q.shape[1] * 8
    out = np.empty((R, N), np.uint8)
    lib().ksqo_awq_unpack(_p(q), _p(out), _sz(R), _sz(N))
    return out


def awq_pack(codes):
    c = _c(codes, np.uint8)
    R, N = c.shape
    out = np.empty((R, N // 8), np.uint32)
    lib().ksqo_awq_pack(_p(c), _p(out), _sz(R), _sz(N))
    return out


def pack_int8_to_int4x2(w):
    w = _c(w, np.int8)
    K, N = w.shape
    out = np.empty((K, N // 2), np.int8)
    lib().ksqo_pack_int8_to_int4x2(_p(w), _p(out), _sz(K), _sz(N))
    return out


def moe_unpack(w):
    """[E, N, K/2] u8 -> codes [E, K, N] u8."""
    w = _c(w, np.uint8)
    E, N, K2 = w.shape
    out = np.empty((E, K2 * 2, N), np.uint8)
    lib().ksqo_moe_unpack(_p(w), _p(out), _sz(E), _sz(N), _sz(K2 * 2))
    return out


def moe_pack(codes):
    """codes [E, K, N] u8 -> [E, N, K/2] u8."""
    c = _c(codes, np.uint8)
    E, K, N = c.shape
    out = np.empty((E, N, K // 2), np.uint8)
    lib().ksqo_moe_pack(_p(c), _p(out), _sz(E), _sz(N), _sz(K))
    return out


def marlin_gptq_repack(qweight):
    q = _c(qweight, np.uint32)
    K, N = q.shape[0] * 8, q.shape[1]
    out = np.empty((K // 16, 2 * N), np.uint32)
    assert lib().ksqo_marlin_gptq_repack(_p(q), _p(out), _sz(K), _sz(N)) == 0
    return out


def marlin_awq_repack(qweight):
    q = _c(qweight, np.uint32)
    K, N = q.shape[0], q.shape[1] * 8
    out = np.empty((K // 16, 2 * N), np.uint32)
    assert lib().ksqo_marlin_awq_repack(_p(q), _p(out), _sz(K), _sz(N)) == 0
    return out


def marlin_awq_zero_points(qz):
    q = _c(qz, np.uint32)
    R, N = q.shape[0], q.shape[1] * 8
    out = np.empty((R, N // 8), np.uint32)
    assert lib().ksqo_marlin_awq_zero_points(_p(q), _p(out), _sz(R), _sz(N)) == 0
    return out


# ---------------------------------------------------------------- W4A16
def w4a16_dequant(codes, scales_bits, zeros, group, dtype):
    c = _c(codes, np.uint8)
    K, N = c.shape
    s = _c(scales_bits, _store_dt(dtype))
    z = None if zeros is None else _c(zeros, np.uint8)
    w = np.empty((K, N), np.float32)
    lib().ksqo_w4a16_dequant(_p(c), _p(s), _p(z) if z is not None else None, _p(w), _sz(K), _sz(N), _sz(group),
                             ctypes.c_int(dtype))
    return w


def gemm_xw_f32(x_bits, w, dtype):
    x = _c(x_bits, _store_dt(dtype))
    w = _c(w, np.float32)
    M, K = x.shape
    N = w.shape[1]
    y = np.empty((M, N), np.float32)
    lib().ksqo_gemm_xw_f32(_p(x), _p(w), _p(y), _sz(M), _sz(N), _sz(K), ctypes.c_int(dtype))
    return y


def gemm_xw_f64(x_bits, w, dtype):
    x = _c(x_bits, _store_dt(dtype))
    w = _c(w, np.float32)
    M, K = x.shape
    N = w.shape[1]
    y = np.empty((M, N), np.float64)
    lib().ksqo_gemm_xw_f64(_p(x), _p(w), _p(y), _sz(M), _sz(N), _sz(K), ctypes.c_int(dtype))
    return y


def w4a16_gemm(x_bits, codes, scales_bits, zeros, group, dtype):
    """Dequantize-then-GEMM, fp32 result (not rounded to dtype)."""
    x = _c(x_bits, _store_dt(dtype))
    c = _c(codes, np.uint8)
    s = _c(scales_bits, _store_dt(dtype))
    z = None if zeros is None else _c(zeros, np.uint8)
    M, K = x.shape
    N = c.shape[1]
    y = np.empty((M, N), np.float32)
    rc = lib().ksqo_w4a16_gemm(_p(x), _p(c), _p(s), _p(z) if z is not None else None, _p(y), _sz(M), _sz(N), _sz(K),
                               _sz(group), ctypes.c_int(dtype))
    assert rc == 0
    return y


# ---------------------------------------------------------------- FP8
def fp8_group_quant(x_bits, k, group, column_major, fuse_silu_mul, dtype):
    x = _c(x_bits, _store_dt(dtype))
    m = x.shape[0]
    q = np.empty((m, k), np.uint8)
    ng = k // group
    s = np.empty((ng, m) if column_major else (m, ng), np.float32)
    lib().ksqo_fp8_group_quant(_p(x), _p(q), _p(s), _sz(m), _sz(k), _sz(group), ctypes.c_int(int(column_major)),
                               ctypes.c_int(int(fuse_silu_mul)), ctypes.c_int(dtype))
    return q, s


def fp8_channel_quant(x_bits, dtype, scale=None):
    """[channels, size] T bits -> (codes, scales); scale given = static quantization."""
    x = _c(x_bits, _store_dt(dtype))
    channels, size = x.shape
    q = np.empty((channels, size), np.uint8)
    static = scale is not None
    s = _c(scale, np.float32).copy() if static else np.empty(channels, np.float32)
    lib().ksqo_fp8_channel_quant(_p(x), _p(q), _p(s), _sz(channels), _sz(size), ctypes.c_int(int(static)),
                                 ctypes.c_int(dtype))
    return q, s


def fp8_tensor_gemm(a, a_scale, b, b_scale):
    a = _c(a, np.uint8)
    b = _c(b, np.uint8)
    m, k = a.shape
    n = b.shape[0]
    out = np.empty((m, n), np.float32)
    lib().ksqo_fp8_tensor_gemm(_p(a), ctypes.c_float(float(a_scale)), _p(b), ctypes.c_float(float(b_scale)), _p(out),
                               _sz(m), _sz(n), _sz(k))
    return out


def fp8_blockwise_gemm(a, a_s, b, b_s, a_s_column_major=True):
    a = _c(a, np.uint8)
    b = _c(b, np.uint8)
    a_s = _c(a_s, np.float32)
    b_s = _c(b_s, np.float32)
    m, k = a.shape
    n = b.shape[0]
    out = np.empty((m, n), np.float32)
    lib().ksqo_fp8_blockwise_gemm(_p(a), _p(a_s), _p(b), _p(b_s), _p(out), _sz(m), _sz(n), _sz(k),
                                  ctypes.c_int(int(a_s_column_major)))
    return out


def fp8_block_quant_weight(w):
    w = _c(w, np.float32)
    n, k = w.shape
    q = np.empty((n, k), np.uint8)
    s = np.empty(((n + 127) // 128, (k + 127) // 128), np.float32)
    lib().ksqo_fp8_block_quant_weight(_p(w), _p(q), _p(s), _sz(n), _sz(k))
    return q, s


# ---------------------------------------------------------------- MoE
def moe_align(topk_ids, E, block_size):
    ids = _c(topk_ids, np.int32).reshape(-1)
    numel = ids.size
    cap = numel + E * (block_size - 1)
    sorted_ids = np.empty(cap, np.int32)
    expert_ids = np.full((cap + block_size - 1) // block_size, -1, np.int32)
    npp = np.zeros(1, np.int32)
    assert lib().ksqo_moe_align(_p(ids), _sz(numel), ctypes.c_int(E), ctypes.c_int(block_size), _p(sorted_ids),
                                _p(expert_ids), _p(npp)) == 0
    return sorted_ids, expert_ids, int(npp[0])


def moe_w4a16_gemm(x_bits, w, scales_bits, topk_ids, topk_w, top_k_div, group, mul_routed, dtype):
    x = _c(x_bits, _store_dt(dtype))
    w = _c(w, np.uint8)
    s = _c(scales_bits, _store_dt(dtype))
    ids = _c(topk_ids, np.int32).reshape(-1)
    tw = _c(topk_w, np.float32).reshape(-1)
    E, N, K2 = w.shape
    K = K2 * 2
    out = np.empty((ids.size, N), np.float32)
    lib().ksqo_moe_w4a16_gemm(_p(x), _p(w), _p(s), _p(ids), _p(tw), _p(out), _sz(ids.size), ctypes.c_int(top_k_div),
                              _sz(N), _sz(K), _sz(group), ctypes.c_int(int(mul_routed)), ctypes.c_int(dtype))
    return out


def moe_topk_softmax(gating, top_k, norm, scaling, dtype):
    g = _c(gating, _store_dt(dtype))
    T, E = g.shape
    w = np.empty((T, top_k), np.float32)
    ids = np.empty((T, top_k), np.int32)
    lib().ksqo_moe_topk_softmax(_p(g), _p(w), _p(ids), _sz(T), _sz(E), _sz(top_k), ctypes.c_int(int(norm)),
                                ctypes.c_float(scaling), ctypes.c_int(dtype))
    return w, ids


def moe_grouped_topk(gating, bias, top_k, groups, topk_group, sigmoid, renorm, scaling, dtype):
    g = _c(gating, _store_dt(dtype))
    T, E = g.shape
    w = np.empty((T, top_k), np.float32)
    ids = np.empty((T, top_k), np.int32)
    b = None if bias is None else _c(bias, np.float32)
    lib().ksqo_moe_grouped_topk(_p(g), None if b is None else _p(b), _p(w), _p(ids), _sz(T), _sz(E), _sz(top_k),
                                _sz(groups), _sz(topk_group), ctypes.c_int(int(sigmoid)), ctypes.c_int(int(renorm)),
                                ctypes.c_float(scaling), ctypes.c_int(dtype))
    return w, ids


def silu_mul(x_bits, dtype):
    x = _c(x_bits, _store_dt(dtype))
    rows, two_i = x.shape
    out = np.empty((rows, two_i // 2), _store_dt(dtype))
    lib().ksqo_silu_mul(_p(x), _p(out), _sz(rows), _sz(two_i // 2), ctypes.c_int(dtype))
    return out


def moe_sum(x_bits, dtype):
    x = _c(x_bits, _store_dt(dtype))
    T, topk, d = x.shape
    out = np.empty((T, d), _store_dt(dtype))
    lib().ksqo_moe_sum(_p(x), _p(out), _sz(T), _sz(topk), _sz(d), ctypes.c_int(dtype))
    return out


def moe_forward(x_bits, w13, s13, w2, s2, topk_ids, topk_w, group, dtype, sum_fp32=False):
    """Whole int4 MoE block as S/kernels/nvidia/moe_kernel_wrapper.cpp:616-652 sequences it:
    GEMM1 (no routed weight) -> T, silu*mul -> T, GEMM2 (* routed weight) -> T, sum over top-k in T (bit patterns of T).
    sum_fp32: the last two steps without their roundings - the second GEMM's fp32 rows summed over top-k, returned as
    fp32 values: the fp32-accumulated reference of a second GEMM that carries the sum."""
    T, topk = np.asarray(topk_ids).shape
    c1 = moe_w4a16_gemm(x_bits, w13, s13, topk_ids, topk_w, topk, group, False, dtype)
    c1b = to_bits(c1, dtype)
    c2b = silu_mul(c1b, dtype)
    c3 = moe_w4a16_gemm(c2b, w2, s2, topk_ids, topk_w, 1, group, True, dtype)
    if sum_fp32:
        return np.asarray(c3, np.float64).reshape(T, topk, -1).sum(1).astype(np.float32)
    c3b = to_bits(c3, dtype).reshape(T, topk, -1)
    return moe_sum(c3b, dtype)


def moe_fp8_forward(x_bits, w13, w13_scale, w2, w2_scale, topk_ids, topk_w, dtype):
    """Whole block-fp8 MoE block as S/kernels/nvidia/moe_kernel_wrapper.cpp:435-456 and 616-652 sequence it: quantize the
    hidden states per token and 128 channels, GEMM1 per expert (no routed weight) -> T, silu*mul fused into the second
    quantization, GEMM2 (* routed weight) -> T, sum over top-k in T.  Built from the functions above, expert by expert."""
    ids = np.asarray(topk_ids)
    T, topk = ids.shape
    E, two_inter, hidden = w13.shape
    inter = two_inter // 2
    a1_q, a1_s = fp8_group_quant(x_bits, hidden, 128, False, False, dtype)
    c1 = np.zeros((T * topk, two_inter), np.float32)
    flat = ids.reshape(-1)
    for e in range(E):
        slots = np.nonzero(flat == e)[0]
        if slots.size:
            rows = slots // topk
            c1[slots] = fp8_blockwise_gemm(a1_q[rows], a1_s[rows], w13[e], w13_scale[e], False)
    c1b = to_bits(c1, dtype)
    a2_q, a2_s = fp8_group_quant(c1b, inter, 128, False, True, dtype)
    c3 = np.zeros((T * topk, hidden), np.float32)
    tw = np.asarray(topk_w, np.float32).reshape(-1)
    for e in range(E):
        slots = np.nonzero(flat == e)[0]
        if slots.size:
            c3[slots] = fp8_blockwise_gemm(a2_q[slots], a2_s[slots], w2[e], w2_scale[e], False) * tw[slots, None]
    c3b = to_bits(c3, dtype).reshape(T, topk, -1)
    return moe_sum(c3b, dtype)


def gptq_act_order_gemm(x_bits, codes, scales_bits, g_idx, dtype, zeros=None):
    """GPTQ with act-order, by its definition: input channel k belongs to quantization group g_idx[k], so
    W[k, n] = (code[k, n] - zp[g_idx[k], n]) * scale[g_idx[k], n] (zp = 8 without zero points) and y = x . W.
    The reference reaches the same product by sorting the rows by g_idx and permuting the activations
    (S/models/quant/marlin_utils.cpp:106-122, K/gptq_marlin/gptq_marlin.cu act_order path); this function does neither.
    numpy, double accumulation: for test sizes."""
    x = from_bits(np.asarray(x_bits), dtype).astype(np.float64)
    sc = from_bits(np.asarray(scales_bits), dtype).astype(np.float64)
    g = np.asarray(g_idx).astype(np.int64)
    z = 8.0 if zeros is None else np.asarray(zeros).astype(np.float64)[g]
    w = (np.asarray(codes).astype(np.float64) - z) * sc[g]
    return (x @ w).astype(np.float32)


def fp8_repack_weight(w):
    """Packed fragment layout of an e4m3 weight [N, K] or [E, N, K] (uint8), as include/ksq.h defines it: fragments of
    16 rows x 128 k in (e, n/16, k/128) order; inside, half h, lane l = 16*((k%128)/32) + n%16, 16 bytes k%32 in
    [16h, 16h+16).  Written as an index permutation in numpy (the layout has no counterpart in the reference)."""
    w = np.asarray(w, np.uint8)
    shape = w.shape
    w3 = w.reshape((-1,) + shape[-2:])
    E, N, K = w3.shape
    # axes: e, nt, r(16), kb, q(4), h(2), byte(16)  ->  e, nt, kb, h, q, r, byte
    v = w3.reshape(E, N // 16, 16, K // 128, 4, 2, 16).transpose(0, 1, 3, 5, 4, 2, 6)
    return np.ascontiguousarray(v).reshape(shape)


# ---------------------------------------------------------------- W4A8
def w4a8_unpack_int4(w):
    """[K, N/2] packed bytes -> [K, N] int8 (low nibble = even column, sign-extended)."""
    w = _c(w, np.int8)
    K, half = w.shape
    out = np.empty((K, 2 * half), np.int8)
    lib().ksqo_w4a8_unpack_int4(_p(w), _p(out), _sz(K), _sz(2 * half))
    return out


def w4a8_static_quant(x_bits, scale, per_channel, dtype, per_token=False):
    x = _c(x_bits, _store_dt(dtype))
    m, k = x.shape
    s = _c(np.asarray(scale, np.float32).reshape(-1), np.float32)
    assert s.size == (k if per_channel else (m if per_token else 1))
    q = np.empty((m, k), np.uint8)
    lib().ksqo_w4a8_static_quant(_p(x), _p(s), _p(q), _sz(m), _sz(k), ctypes.c_int(1 if per_channel else (3 if per_token else 0)),
                                 ctypes.c_int(dtype))
    return q


def w4a8_group_sums(q, group=128):
    q = _c(q, np.uint8)
    m, k = q.shape
    out = np.empty((m, k // group), np.float32)
    lib().ksqo_w4a8_group_sums_g(_p(q), _p(out), _sz(m), _sz(k), _sz(group))
    return out


def w4a8_gemm(a_q, w, scales_f16_bits, alpha, group=128):
    a = _c(a_q, np.uint8)
    w = _c(w, np.int8)
    s = _c(scales_f16_bits, np.uint16)
    m, k = a.shape
    n = 2 * w.shape[1]
    assert w.shape[0] == k and s.shape == (k // group, n)
    out = np.empty((m, n), np.float32)
    lib().ksqo_w4a8_gemm(_p(a), _p(w), _p(s), ctypes.c_float(float(alpha)), _p(out), _sz(m), _sz(n), _sz(k),
                         _sz(group))
    return out


def w4a8_repack_weight(w):
    """Packed fragment layout of a W4A8 weight ([K, N/2] packed int4) as include/ksq.h defines it, returned as uint32
    words: fragment (n/16, k/128) of 256 words; word 4*lane + i of lane = 16*((k%128)/32) + n%16 holds the codes
    u = w + 8 of k%32 in [8i, 8i+8): nibble 2j = element j, nibble 2j+1 = element 4+j.  numpy index arithmetic (the
    layout has no counterpart in the reference)."""
    u = (w4a8_unpack_int4(w).astype(np.int32) + 8).astype(np.uint32)  # [K, N]
    K, N = u.shape
    # axes: kb, q(4), i(4), e(8), nt, r(16)  ->  nt, kb, q, r, i, e
    v = u.reshape(K // 128, 4, 4, 8, N // 16, 16).transpose(4, 0, 1, 5, 2, 3)
    pos = np.array([0, 2, 4, 6, 1, 3, 5, 7], np.uint32) * 4
    words = (v << pos).sum(axis=-1, dtype=np.uint64).astype(np.uint32)
    return np.ascontiguousarray(words).reshape(-1)


def moe_act_order_forward(x_bits, codes13, s13_bits, g13, codes2, s2_bits, g2, topk_ids, topk_w, dtype):
    """Int4 MoE block with act-order (desc_act) experts, by the definition of g_idx: row k of expert e belongs to
    quantization group g[e, k], W_e[k, n] = (code[e, k, n] - 8) * scale[e, g[e, k], n] (codes [E, K, N] in checkpoint row
    order, scales [E, K/group, N]).  The reference reaches the same products by sorting each expert's rows by group and
    permuting the activations (S/layers/nvidia/marlin_moe_layer.cpp:71-93); this function does neither.  Rounding as in
    moe_forward: GEMM1 -> T, silu*mul -> T, GEMM2 * routed weight -> T, sum over top-k in T.  numpy, for test sizes."""
    ids = np.asarray(topk_ids)
    tw = np.asarray(topk_w, np.float32)
    T, topk = ids.shape
    x = from_bits(np.asarray(x_bits), dtype).astype(np.float64)

    def dense(codes, s_bits, g):
        s = from_bits(np.asarray(s_bits), dtype).astype(np.float64)
        E = codes.shape[0]
        return [(np.asarray(codes[e]).astype(np.float64) - 8.0) * s[e][np.asarray(g[e]).astype(np.int64)] for e in range(E)]

    w13, w2 = dense(codes13, s13_bits, g13), dense(codes2, s2_bits, g2)
    c1 = np.stack([x[t] @ w13[ids[t, j]] for t in range(T) for j in range(topk)]).astype(np.float32)
    c2b = silu_mul(to_bits(c1, dtype), dtype)
    c2 = from_bits(c2b, dtype).astype(np.float64)
    c3 = np.stack([(c2[t * topk + j] @ w2[ids[t, j]]).astype(np.float32) * tw[t, j]
                   for t in range(T) for j in range(topk)]).astype(np.float32)
    return moe_sum(to_bits(c3, dtype).reshape(T, topk, -1), dtype)
