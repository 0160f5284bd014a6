"""Host-side mirror of the reference's kernel-wrapper surface for the quantized-GEMM path, on torch device tensors.

Each function names the ``Invoke*`` wrapper of the reference it stands for
(src/ksana_llm/kernels/nvidia/basic_kernel_wrapper.h:32-115,295-336 and moe_kernel_wrapper.h:28-88) and forwards to
the C-ABI of libksq_hip.so on the tensor's current stream.  Torch is used for device memory and streams only.
"""
import torch

from . import lib as _l

_lib = _l.load()

F16, BF16 = _l.F16, _l.BF16


def _dt(t, allow_f32=False):
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.bfloat16:
        return BF16
    if allow_f32 and t.dtype == torch.float32:   # the block-fp8 quantizer and GEMM also take / give fp32 activations
        return _l.F32
    raise TypeError("activation dtype must be float16 or bfloat16, got %s" % t.dtype)


def _torch_dt(tag):
    return torch.float16 if tag == F16 else torch.bfloat16


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensor required"
    return t.data_ptr()


# ----------------------------------------------------------------------------------------------- load-time repack
def _need_bytes(t, nbytes, what):
    """The C-ABI takes bare pointers: a tensor that is smaller than the layout it is declared to hold would be read
    past its end on the device, so the wrappers check the size here."""
    have = t.numel() * t.element_size()
    if have < nbytes:
        raise ValueError("%s: tensor holds %d bytes, the declared layout needs %d" % (what, have, nbytes))


def repack_weight(src, layout, E, K, N):
    """Checkpoint int4 weight -> CDNA4 tile layout (uint8 tensor of E*K*N/2 bytes)."""
    _need_bytes(src, E * K * N // 2, "repack_weight")
    dst = torch.empty(_lib.ksq_w4a16_packed_weight_bytes(E, K, N), dtype=torch.uint8, device=src.device)
    _l.check(_lib.ksq_w4a16_repack(_ptr(src), layout, _ptr(dst), E, K, N, _stream()))
    return dst


def unpack_weight(packed, layout, E, K, N):
    """Inverse of :func:`repack_weight`; returns the checkpoint layout as int32 (GPTQ/AWQ) or uint8/int8 bytes."""
    if layout == _l.SRC_GPTQ:
        dst = torch.empty((E, K // 8, N) if E > 1 else (K // 8, N), dtype=torch.int32, device=packed.device)
    elif layout == _l.SRC_AWQ:
        dst = torch.empty((E, K, N // 8) if E > 1 else (K, N // 8), dtype=torch.int32, device=packed.device)
    elif layout == _l.SRC_MOE_NK:
        dst = torch.empty((E, N, K // 2), dtype=torch.uint8, device=packed.device)
    else:
        dst = torch.empty((E, K, N // 2) if E > 1 else (K, N // 2), dtype=torch.int8, device=packed.device)
    _l.check(_lib.ksq_w4a16_unpack(_ptr(packed), layout, _ptr(dst), E, K, N, _stream()))
    return dst


def repack_scales(src, layout, E, K, N, group):
    _need_bytes(src, E * (K // group) * N * src.element_size(), "repack_scales")
    dst = torch.empty(E * (K // group) * N, dtype=src.dtype, device=src.device)
    _l.check(_lib.ksq_w4a16_repack_scales(_ptr(src), layout, _ptr(dst), E, K, N, group, _dt(src), _stream()))
    return dst


def unpack_scales(packed, layout, E, K, N, group):
    G = K // group
    shape = ((E, G, N) if E > 1 else (G, N)) if layout == _l.SCALE_GN else (E, N, G)
    dst = torch.empty(shape, dtype=packed.dtype, device=packed.device)
    _l.check(_lib.ksq_w4a16_unpack_scales(_ptr(packed), layout, _ptr(dst), E, K, N, group, _dt(packed), _stream()))
    return dst


def repack_zeros(src, layout, K, N, group):
    _need_bytes(src, (K // group) * N // (2 if layout == _l.ZERO_AWQ_PACKED else 1), "repack_zeros")
    dst = torch.empty((K // group) * N, dtype=torch.uint8, device=src.device)
    _l.check(_lib.ksq_w4a16_repack_zeros(_ptr(src), layout, _ptr(dst), K, N, group, _stream()))
    return dst


def unpack_zeros(packed, layout, K, N, group):
    G = K // group
    if layout == _l.ZERO_AWQ_PACKED:
        dst = torch.empty((G, N // 8), dtype=torch.int32, device=packed.device)
    else:
        dst = torch.empty((G, N), dtype=torch.uint8, device=packed.device)
    _l.check(_lib.ksq_w4a16_unpack_zeros(_ptr(packed), layout, _ptr(dst), K, N, group, _stream()))
    return dst


# ----------------------------------------------------------------------------------------------- W4A16 GEMM
def w4a16_workspace_size(max_m, n, k, group, dtype):
    return _lib.ksq_w4a16_workspace_size(max_m, n, k, group, dtype)


_WORKSPACES = {}


def _w4a16_workspace(device, m, n, k, group, dt):
    """A per-device scratch tensor large enough for this call (grown on demand, like the engine's shared workspace)."""
    need = _lib.ksq_w4a16_workspace_size(m, n, k, group, dt)
    if need == 0:
        return None
    cur = _WORKSPACES.get(device)
    if cur is None or cur.numel() < need:
        cur = torch.empty(need, dtype=torch.uint8, device=device)
        _WORKSPACES[device] = cur
    return cur


def w4a16_gemm(x, w_packed, scales_packed, zeros_packed, n, k, group, out=None, workspace=None):
    """InvokeFpAIntBGroupCudaGemm / InvokeFpAIntBGroupCutlassGemm / InvokeMarlinGemm / InvokeMacheteGemm."""
    m = x.shape[0]
    _need_bytes(x, m * k * 2, "w4a16_gemm: x")
    _need_bytes(w_packed, k * n // 2, "w4a16_gemm: packed weight")
    _need_bytes(scales_packed, (k // group) * n * 2, "w4a16_gemm: scales")
    if zeros_packed is not None:
        _need_bytes(zeros_packed, (k // group) * n, "w4a16_gemm: zero points")
    if out is None:
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    if workspace is None:
        workspace = _w4a16_workspace(x.device, m, n, k, group, _dt(x))
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _l.check(_lib.ksq_w4a16_gemm(_ptr(out), _ptr(x), _ptr(w_packed), _ptr(scales_packed), _ptr(zeros_packed),
                                 _ptr(workspace), ws_bytes, m, n, k, group, _dt(x), _stream()))
    return out


def w4a16_gemm_f32(x, w_packed, scales_packed, zeros_packed, n, k, group, workspace=None):
    """ksq_w4a16_gemm_f32: the same kernels and plan as w4a16_gemm with the fp32 sums stored unrounded (verification)."""
    m = x.shape[0]
    _need_bytes(x, m * k * 2, "w4a16_gemm_f32: x")
    _need_bytes(w_packed, k * n // 2, "w4a16_gemm_f32: packed weight")
    _need_bytes(scales_packed, (k // group) * n * 2, "w4a16_gemm_f32: scales")
    out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    if workspace is None:
        workspace = _w4a16_workspace(x.device, m, n, k, group, _dt(x))
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _l.check(_lib.ksq_w4a16_gemm_f32(_ptr(out), _ptr(x), _ptr(w_packed), _ptr(scales_packed), _ptr(zeros_packed),
                                     _ptr(workspace), ws_bytes, m, n, k, group, _dt(x), _stream()))
    return out


# ----------------------------------------------------------------------------------------------- FP8
def per_token_group_quant_fp8(x, k, group=128, column_major=True, fuse_silu_mul=False, q=None, s=None):
    """InvokePerTokenGroupQuantFp8E4m3: returns (codes uint8 [m,k], scales fp32 [k/group,m] or [m,k/group])."""
    m = x.shape[0]
    if q is None:
        q = torch.empty((m, k), dtype=torch.uint8, device=x.device)
    if s is None:
        s = torch.empty((k // group, m) if column_major else (m, k // group), dtype=torch.float32, device=x.device)
    _l.check(_lib.ksq_fp8_group_quant(_ptr(x), _ptr(q), _ptr(s), m, k, group, int(column_major), int(fuse_silu_mul),
                                      _dt(x, allow_f32=True), _stream()))
    return q, s


def fp8_blockwise_gemm(a_q, a_s, b, b_s, out_dtype=torch.bfloat16, out=None, workspace=None):
    """InvokeBlockGemm / DeepGEMMWrapper::Gemm: a_q [m,k] e4m3 bytes, a_s [k/128,m], b [n,k] packed by
    fp8_repack_weight, b_s [n/128,k/128]."""
    m, k = a_q.shape
    n = b.shape[0]
    _need_bytes(a_s, (k // 128) * m * 4, "fp8_blockwise_gemm: activation scales")
    _need_bytes(b, n * k, "fp8_blockwise_gemm: weight")
    _need_bytes(b_s, ((n + 127) // 128) * (k // 128) * 4, "fp8_blockwise_gemm: weight scales")
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a_q.device)
    if workspace is None:
        need = _lib.ksq_fp8_blockwise_workspace_size(m, n, k)
        if need:
            workspace = _WORKSPACES.get(a_q.device)
            if workspace is None or workspace.numel() < need:
                workspace = _WORKSPACES[a_q.device] = torch.empty(need, dtype=torch.uint8, device=a_q.device)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _l.check(_lib.ksq_fp8_blockwise_gemm(_ptr(a_q), _ptr(a_s), _ptr(b), _ptr(b_s), _ptr(out), m, n, k,
                                         _dt(out, allow_f32=True), _ptr(workspace), ws_bytes, _stream()))
    return out


def fp8_blockwise_gemm_f32(a_q, a_s, b, b_s, workspace=None):
    """ksq_fp8_blockwise_gemm_f32: the same kernels and plan as fp8_blockwise_gemm with the fp32 sums stored unrounded."""
    m, k = a_q.shape
    n = b.shape[0]
    _need_bytes(a_s, (k // 128) * m * 4, "fp8_blockwise_gemm_f32: activation scales")
    _need_bytes(b, n * k, "fp8_blockwise_gemm_f32: weight")
    _need_bytes(b_s, ((n + 127) // 128) * (k // 128) * 4, "fp8_blockwise_gemm_f32: weight scales")
    out = torch.empty((m, n), dtype=torch.float32, device=a_q.device)
    if workspace is None:
        need = _lib.ksq_fp8_blockwise_workspace_size(m, n, k)
        if need:
            workspace = _WORKSPACES.get(a_q.device)
            if workspace is None or workspace.numel() < need:
                workspace = _WORKSPACES[a_q.device] = torch.empty(need, dtype=torch.uint8, device=a_q.device)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    _l.check(_lib.ksq_fp8_blockwise_gemm_f32(_ptr(a_q), _ptr(a_s), _ptr(b), _ptr(b_s), _ptr(out), m, n, k,
                                             _ptr(workspace), ws_bytes, _stream()))
    return out


# ----------------------------------------------------------------------------------------------- MoE
def moe_align_block_size(topk_ids, num_experts, block_m):
    """InvokeSglMoeAlignBlockSize / InvokeMoeAlignBlockSize: (sorted_ids, expert_ids, num_post_pad) int32 tensors."""
    ids = topk_ids.reshape(-1)
    numel = ids.numel()
    cap = _lib.ksq_moe_align_capacity(numel, num_experts, block_m)
    dev = topk_ids.device
    sorted_ids = torch.empty(cap, dtype=torch.int32, device=dev)
    expert_ids = torch.empty((cap + block_m - 1) // block_m, dtype=torch.int32, device=dev)
    num_post_pad = torch.empty(1, dtype=torch.int32, device=dev)
    scratch = torch.empty(_lib.ksq_moe_align_scratch_bytes(numel, num_experts), dtype=torch.uint8, device=dev)
    _l.check(_lib.ksq_moe_align(_ptr(ids), numel, num_experts, block_m, _ptr(sorted_ids), _ptr(expert_ids),
                                _ptr(num_post_pad), _ptr(scratch), _stream()))
    return sorted_ids, expert_ids, num_post_pad


def moe_w4a16_gemm(x, w_packed, scales_packed, topk_w, sorted_ids, expert_ids, num_post_pad, numel, top_k, E, n, k,
                   group, block_m, out=None):
    """InvokeMoeWna16Gemm / InvokeFusedMoeGptqAwqKernel: out [numel, n]."""
    _need_bytes(x, ((numel + top_k - 1) // top_k) * k * 2, "moe_w4a16_gemm: x")
    _need_bytes(w_packed, E * k * n // 2, "moe_w4a16_gemm: packed weight")
    _need_bytes(scales_packed, E * (k // group) * n * 2, "moe_w4a16_gemm: scales")
    if out is None:
        out = torch.empty((numel, n), dtype=x.dtype, device=x.device)
    _l.check(_lib.ksq_moe_w4a16_gemm(_ptr(out), _ptr(x), _ptr(w_packed), _ptr(scales_packed), None, _ptr(topk_w),
                                     _ptr(sorted_ids), _ptr(expert_ids), _ptr(num_post_pad), numel, top_k, E, n, k,
                                     group, block_m, _dt(x), _stream()))
    return out


def moe_w4a16_gate_up_silu(x, w_packed, scales_packed, sorted_ids, expert_ids, num_post_pad, numel, top_k, E, n, k, group,
                           block_m, out=None):
    """The first MoE GEMM with silu*mul in its epilogue (any block size of moe_w4a16_gemm): out [numel, n/2], bit for bit what
    moe_w4a16_gemm followed by silu_and_mul gives."""
    _need_bytes(x, ((numel + top_k - 1) // top_k) * k * 2, "moe_w4a16_gate_up_silu: x")
    _need_bytes(w_packed, E * k * n // 2, "moe_w4a16_gate_up_silu: packed weight")
    _need_bytes(scales_packed, E * (k // group) * n * 2, "moe_w4a16_gate_up_silu: scales")
    if out is None:
        out = torch.empty((numel, n // 2), dtype=x.dtype, device=x.device)
    _l.check(_lib.ksq_moe_w4a16_gate_up_silu(_ptr(out), _ptr(x), _ptr(w_packed), _ptr(scales_packed), None,
                                             _ptr(sorted_ids), _ptr(expert_ids), _ptr(num_post_pad), numel, top_k, E, n,
                                             k, group, block_m, _dt(x), _stream()))
    return out


def moe_topk_softmax(gating, top_k, norm_topk_prob=False, routed_scaling_factor=1.0):
    """InvokeBasicSoftmaxTopk: (topk_weights fp32 [T, top_k], topk_ids int32 [T, top_k])."""
    tokens, E = gating.shape
    dt = _l.F32 if gating.dtype == torch.float32 else _dt(gating)
    w = torch.empty((tokens, top_k), dtype=torch.float32, device=gating.device)
    ids = torch.empty((tokens, top_k), dtype=torch.int32, device=gating.device)
    _l.check(_lib.ksq_moe_topk_softmax(_ptr(gating), _ptr(w), _ptr(ids), tokens, E, top_k, int(norm_topk_prob),
                                       float(routed_scaling_factor), dt, _stream()))
    return w, ids


def moe_grouped_topk(gating, top_k, num_expert_group=1, topk_group=1, scoring_func="softmax", e_bias=None,
                     renormalize=False, routed_scaling_factor=1.0):
    """InvokeGroupedTopk: (topk_weights fp32 [T, top_k], topk_ids int32 [T, top_k]); e_bias fp32 [E] or None."""
    tokens, E = gating.shape
    if scoring_func not in ("softmax", "sigmoid"):
        raise ValueError("Unsupported scoring function: %s" % scoring_func)
    dt = _l.F32 if gating.dtype == torch.float32 else _dt(gating)
    w = torch.empty((tokens, top_k), dtype=torch.float32, device=gating.device)
    ids = torch.empty((tokens, top_k), dtype=torch.int32, device=gating.device)
    if e_bias is not None and e_bias.dtype != torch.float32:
        raise ValueError("e_bias must be fp32")
    _l.check(_lib.ksq_moe_grouped_topk(_ptr(gating), _ptr(e_bias) if e_bias is not None else None, _ptr(w), _ptr(ids),
                                       tokens, E, top_k, num_expert_group, topk_group,
                                       1 if scoring_func == "sigmoid" else 0, int(renormalize),
                                       float(routed_scaling_factor), dt, _stream()))
    return w, ids


def silu_and_mul(x, out=None):
    """InvokeSiluAndMul: x [rows, 2*inter] -> [rows, inter]."""
    rows, two = x.shape
    if out is None:
        out = torch.empty((rows, two // 2), dtype=x.dtype, device=x.device)
    _l.check(_lib.ksq_moe_silu_mul(_ptr(x), _ptr(out), rows, two // 2, _dt(x), _stream()))
    return out


def moe_sum(x, out=None):
    """InvokeMoeSum: x [tokens, topk, d] -> [tokens, d]."""
    tokens, topk, d = x.shape
    if out is None:
        out = torch.empty((tokens, d), dtype=x.dtype, device=x.device)
    _l.check(_lib.ksq_moe_sum(_ptr(x), _ptr(out), tokens, topk, d, _dt(x), _stream()))
    return out


# up to this many tokens the int4 MoE block runs its two-launch form (ksq_moe_w4a16_down_sum).  DeepSeek-V3 expert shapes,
# whole block with / without it: 1 token 39.5 / 49.5 us, 2 68 / 74, 3 98.5 / 103.5, 4 128 / 135, 8 230 / 211
FEW_TOKENS = 4


def fused_moe_w4a16(x, w13_packed, s13_packed, w2_packed, s2_packed, topk_ids, topk_w, E, hidden, inter, group,
                    block_m=None):
    """InvokeFusedMoe<T,false> for int4 weights (S/kernels/nvidia/moe_kernel_wrapper.cpp:463-654):
    align -> GEMM1 -> silu*mul -> GEMM2 (* routed weight) -> sum over top-k."""
    T, topk = topk_ids.shape
    numel = T * topk
    tw = topk_w.reshape(-1).to(torch.float32).contiguous()
    if block_m is None and T <= FEW_TOKENS and numel <= 64 and topk <= 32 and (2 * inter) % 32 == 0:
        # a few decode tokens: two launches - the first GEMM with every slot a block of its own (no aligned
        # permutation) and the activation in its epilogue, the second with the sum over top-k in it
        ids = topk_ids.reshape(-1).to(torch.int32).contiguous()
        c2 = torch.empty((numel, inter), dtype=x.dtype, device=x.device)
        _l.check(_lib.ksq_moe_w4a16_gate_up_silu(_ptr(c2), _ptr(x), _ptr(w13_packed), _ptr(s13_packed), None, None, _ptr(ids),
                                                 None, numel, topk, E, 2 * inter, hidden, group, 16, _dt(x), _stream()))
        out = torch.empty((T, hidden), dtype=x.dtype, device=x.device)
        _l.check(_lib.ksq_moe_w4a16_down_sum(_ptr(out), _ptr(c2), _ptr(w2_packed), _ptr(s2_packed), _ptr(tw), _ptr(ids), T,
                                             topk, E, hidden, inter, group, _dt(x), _stream()))
        return out
    if block_m is None:
        block_m = _lib.ksq_moe_block_m(numel, E)
    sorted_ids, expert_ids, npp = moe_align_block_size(topk_ids, E, block_m)
    # the activation runs in the first GEMM's epilogue, except with 128-row blocks (a size ksq_moe_block_m no longer
    # picks but a caller may ask for), where the two launches measured faster (64 rows per expert: 1.75 against 1.87 ms)
    if block_m != 128 and (2 * inter) % 32 == 0:
        c2 = moe_w4a16_gate_up_silu(x, w13_packed, s13_packed, sorted_ids, expert_ids, npp, numel, topk, E, 2 * inter,
                                    hidden, group, block_m)
    else:
        c1 = moe_w4a16_gemm(x, w13_packed, s13_packed, None, sorted_ids, expert_ids, npp, numel, topk, E, 2 * inter,
                            hidden, group, block_m)
        c2 = silu_and_mul(c1)
    c3 = moe_w4a16_gemm(c2, w2_packed, s2_packed, tw, sorted_ids, expert_ids, npp, numel, 1, E, hidden, inter, group,
                        block_m)
    return moe_sum(c3.view(T, topk, hidden))


def moe_fp8_blockwise_gemm(a_q, a_s, a_s_column_major, b, b_s, topk_w, sorted_ids, expert_ids, num_post_pad, numel,
                           top_k, block_m, out_dtype=torch.bfloat16, out=None):
    """fp8_w8a8 block-quantized fused_moe_kernel launch: a_q [rows,k] e4m3 bytes, b [E,n,k] packed by fp8_repack_weight,
    b_s [E,n/128,k/128]; out [numel, n]."""
    rows, k = a_q.shape
    E, n = b.shape[0], b.shape[1]
    if out is None:
        out = torch.empty((numel, n), dtype=out_dtype, device=a_q.device)
    _l.check(_lib.ksq_moe_fp8_blockwise_gemm(_ptr(out), _ptr(a_q), _ptr(a_s), int(a_s_column_major), rows, _ptr(b),
                                             _ptr(b_s), _ptr(topk_w) if topk_w is not None else None,
                                             _ptr(sorted_ids), _ptr(expert_ids), _ptr(num_post_pad), numel, top_k, E, n,
                                             k, block_m, _dt(out), _stream()))
    return out


def fused_moe_fp8_blockwise(x, w13, w13_scale, w2, w2_scale, topk_ids, topk_w, block_m=None):
    """InvokeFusedMoe<T,false> for block-quantized fp8 experts (S/kernels/nvidia/moe_kernel_wrapper.cpp:463-654 with
    compute_dtype TYPE_BLOCK_FP8_E4M3): quantize x per token and 128 channels -> align -> GEMM1 -> silu*mul fused into
    the second quantization -> GEMM2 (* routed weight) -> sum over top-k.  w13 [E, 2*inter, hidden], w2 [E, hidden, inter]
    e4m3 bytes packed by fp8_repack_weight, scales fp32 per 128 x 128 block."""
    T, topk = topk_ids.shape
    E, two_inter, hidden = w13.shape
    inter = two_inter // 2
    numel = T * topk
    tw = topk_w.reshape(-1).to(torch.float32).contiguous()
    if block_m is None and T <= FEW_TOKENS and numel <= 64 and topk <= 32:
        # a few decode tokens: no aligned permutation, the sum over top-k inside the second GEMM (as fused_moe_w4a16)
        ids = topk_ids.reshape(-1).to(torch.int32).contiguous()
        a1_q, a1_s = per_token_group_quant_fp8(x, hidden, 128, False)
        c1 = moe_fp8_blockwise_gemm(a1_q, a1_s, False, w13, w13_scale, None, None, ids, None, numel, topk, 16, x.dtype)
        a2_q, a2_s = per_token_group_quant_fp8(c1, inter, 128, False, fuse_silu_mul=True)
        out = torch.empty((T, hidden), dtype=x.dtype, device=x.device)
        _l.check(_lib.ksq_moe_fp8_down_sum(_ptr(out), _ptr(a2_q), _ptr(a2_s), _ptr(w2), _ptr(w2_scale), _ptr(tw), _ptr(ids), T,
                                           topk, E, hidden, inter, _dt(out), _stream()))
        return out
    if block_m is None:
        block_m = _lib.ksq_moe_fp8_block_m(numel, E)
    sorted_ids, expert_ids, npp = moe_align_block_size(topk_ids, E, block_m)
    a1_q, a1_s = per_token_group_quant_fp8(x, hidden, 128, False)
    c1 = moe_fp8_blockwise_gemm(a1_q, a1_s, False, w13, w13_scale, None, sorted_ids, expert_ids, npp, numel, topk,
                                block_m, x.dtype)
    a2_q, a2_s = per_token_group_quant_fp8(c1, inter, 128, False, fuse_silu_mul=True)
    c3 = moe_fp8_blockwise_gemm(a2_q, a2_s, False, w2, w2_scale, tw, sorted_ids, expert_ids, npp, numel, 1, block_m,
                                x.dtype)
    return moe_sum(c3.view(T, topk, hidden))


def fp8_e4m3_quantize(x, scale=None):
    """Fp8E4m3Quantize: x [channels, size] -> (codes uint8, scale fp32 [channels]); scale given = static."""
    channels, size = x.shape
    q = torch.empty((channels, size), dtype=torch.uint8, device=x.device)
    static = scale is not None
    s = scale if static else torch.empty(channels, dtype=torch.float32, device=x.device)
    _l.check(_lib.ksq_fp8_channel_quant(_ptr(x), _ptr(q), _ptr(s), channels, size, int(static), _dt(x, allow_f32=True), _stream()))
    return q, s


def fp8_quantized_matmul(a_q, a_scale, b, b_scale, out_dtype=torch.bfloat16, out=None, workspace=None):
    """Fp8QuantizedMatMul: a_q [m,k] e4m3 bytes, b [n,k] packed by fp8_repack_weight, one fp32 device scale each."""
    m, k = a_q.shape
    n = b.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a_q.device)
    if workspace is None:
        workspace = torch.empty(_lib.ksq_fp8_tensor_gemm_workspace_size(m, n, k), dtype=torch.uint8, device=a_q.device)
    _l.check(_lib.ksq_fp8_tensor_gemm(_ptr(a_q), _ptr(a_scale), _ptr(b), _ptr(b_scale), _ptr(out), m, n, k, _dt(out, allow_f32=True),
                                      _ptr(workspace), workspace.numel(), _stream()))
    return out


def sort_g_idx(g_idx):
    """MarlinSortGIdx: perm = stable argsort of the act-order group index (int32 [K], same device)."""
    return torch.argsort(g_idx.to(torch.int64), stable=True).to(torch.int32)


def repack_weight_act_order(qweight, perm, K, N):
    """gptq_marlin_repack with a permutation: qweight [K/8, N] int32 (GPTQ), perm int32 [K] -> packed weight."""
    out = torch.empty(_lib.ksq_w4a16_packed_weight_bytes(1, K, N), dtype=torch.uint8, device=qweight.device)
    _l.check(_lib.ksq_w4a16_repack_act_order(_ptr(qweight), _ptr(perm), _ptr(out), K, N, _stream()))
    return out


def permute_columns(x, perm, out=None):
    """out[r, j] = x[r, perm[j]]."""
    m, k = x.shape
    if out is None:
        out = torch.empty_like(x)
    _l.check(_lib.ksq_permute_columns(_ptr(x), _ptr(perm), _ptr(out), m, k, _dt(x), _stream()))
    return out


def moe_permute_columns(x, perm, topk_ids, top_k, out=None):
    """out[s, j] = x[s // top_k, perm[topk_ids[s], j]]: x [rows, k], perm int32 [E, k], topk_ids int32 [numel]."""
    k = x.shape[1]
    numel = topk_ids.numel()
    if out is None:
        out = torch.empty((numel, k), dtype=x.dtype, device=x.device)
    _l.check(_lib.ksq_moe_permute_columns(_ptr(x), _ptr(perm), _ptr(topk_ids), _ptr(out), numel, k, top_k, perm.shape[0],
                                          _dt(x), _stream()))
    return out


def fp8_repack_weight(w):
    """Checkpoint-layout e4m3 weight [N, K] or [E, N, K] (uint8) -> the packed fragment layout the FP8 GEMMs read."""
    E = w.shape[0] if w.dim() == 3 else 1
    N, K = w.shape[-2], w.shape[-1]
    out = torch.empty_like(w)
    _l.check(_lib.ksq_fp8_repack_weight(_ptr(w), _ptr(out), E, N, K, _stream()))
    return out


def fp8_unpack_weight(packed):
    """Inverse of :func:`fp8_repack_weight` (the tensor keeps the logical shape [N, K] / [E, N, K])."""
    E = packed.shape[0] if packed.dim() == 3 else 1
    N, K = packed.shape[-2], packed.shape[-1]
    out = torch.empty_like(packed)
    _l.check(_lib.ksq_fp8_unpack_weight(_ptr(packed), _ptr(out), E, N, K, _stream()))
    return out


# ----------------------------------------------------------------------------------------------- W4A8
def w4a8_repack_weight(w):
    """W4A8 weight [K, N/2] (int8/uint8, two's-complement nibbles, low nibble = even column: the input of the
    reference's PreprocessWeightsForMixedGemm) -> the packed fragment layout ksq_w4a8_gemm reads."""
    K, half = w.shape
    out = torch.empty(_lib.ksq_w4a8_packed_weight_bytes(2 * half, K), dtype=torch.uint8, device=w.device)
    _l.check(_lib.ksq_w4a8_repack_weight(_ptr(w), _ptr(out), 2 * half, K, _stream()))
    return out


def w4a8_unpack_weight(packed, K, N):
    """Inverse of :func:`w4a8_repack_weight`: uint8 [K, N/2]."""
    out = torch.empty((K, N // 2), dtype=torch.uint8, device=packed.device)
    _l.check(_lib.ksq_w4a8_unpack_weight(_ptr(packed), _ptr(out), N, K, _stream()))
    return out


def w4a8_static_quant(x, scale, per_channel=False, per_token=False, group=128):
    """StaticQuantizeE4M3PerTensor / PerChannel / PerToken: x [m,k] T, scale fp32 [1], [k] or [m] -> (codes uint8
    [m,k], group sums fp32 [k/group, m]); group 128 or 64."""
    m, k = x.shape
    q = torch.empty((m, k), dtype=torch.uint8, device=x.device)
    xsum = torch.empty((k // group, m), dtype=torch.float32, device=x.device)
    mode = _l.W4A8_PER_CHANNEL if per_channel else (_l.W4A8_PER_TOKEN if per_token else _l.W4A8_PER_TENSOR)
    if group == 64:
        mode |= _l.W4A8_SUMS_PER_64
    _l.check(_lib.ksq_w4a8_static_quant(_ptr(x), _ptr(scale), _ptr(q), _ptr(xsum), m, k, mode, _dt(x), _stream()))
    return q, xsum


def w4a8_group_sums(a_q, group=128):
    """Group sums of activations that are e4m3 already (uint8 [m,k]) -> fp32 [k/group, m]; group 128 or 64."""
    m, k = a_q.shape
    xsum = torch.empty((k // group, m), dtype=torch.float32, device=a_q.device)
    mode = _l.W4A8_SUMS_ONLY | (_l.W4A8_SUMS_PER_64 if group == 64 else 0)
    _l.check(_lib.ksq_w4a8_static_quant(_ptr(a_q), None, None, _ptr(xsum), m, k, mode, F16, _stream()))
    return xsum


def w4a8_gemm(a_q, xsum, w_packed, scales, alpha, n, out_dtype=torch.bfloat16, out=None, workspace=None, group=128):
    """FinegrainedMixedDtypeGemmWrapper::Forward: a_q [m,k] e4m3 bytes, xsum [k/group, m], scales fp16 [k/group, n]."""
    m, k = a_q.shape
    _need_bytes(xsum, (k // group) * m * 4, "w4a8_gemm: group sums")
    _need_bytes(w_packed, n * k // 2, "w4a8_gemm: packed weight")
    _need_bytes(scales, (k // group) * n * 2, "w4a8_gemm: scales")
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a_q.device)
    if workspace is None:
        need = _lib.ksq_w4a8_workspace_size(m, n, k)
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=a_q.device)
    assert scales.dtype == torch.float16
    _l.check(_lib.ksq_w4a8_gemm(_ptr(a_q), _ptr(xsum), _ptr(w_packed), _ptr(scales), float(alpha), _ptr(out), m, n, k,
                                group, _dt(out), _ptr(workspace), workspace.numel(), _stream()))
    return out
