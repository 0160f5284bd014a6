"""ctypes binding of libksq_hip.so; signatures follow include/ksq.h one to one."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("KSQ_LIB_PATH", os.path.join(_HERE, "libksq_hip.so"))

F16, BF16, F32 = 0, 1, 2
SRC_GPTQ, SRC_AWQ, SRC_MOE_NK, SRC_INT4X2_KN = 0, 1, 2, 3
SCALE_GN, SCALE_NG = 0, 1
ZERO_AWQ_PACKED, ZERO_U8_GN = 0, 1
KIND_W4A16, KIND_FP8_BLOCKWISE, KIND_MOE_W4A16, KIND_W4A8 = 0, 1, 2, 3
W4A8_PER_TENSOR, W4A8_PER_CHANNEL, W4A8_SUMS_ONLY, W4A8_PER_TOKEN = 0, 1, 2, 3
W4A8_SUMS_PER_64 = 16

c_sz = ctypes.c_size_t
c_p = ctypes.c_void_p
c_i = ctypes.c_int


class TileDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in
                ("kernel", "block_m", "block_n", "block_k", "waves", "split_k", "grid", "x_chunk")]


# name -> (restype, argtypes); also the list the ABI test checks against the header
SIGNATURES = {
    "ksq_version": (c_i, []),
    "ksq_last_error_string": (ctypes.c_char_p, []),
    "ksq_w4a16_packed_weight_bytes": (c_sz, [c_sz, c_sz, c_sz]),
    "ksq_w4a16_packed_scales_bytes": (c_sz, [c_sz, c_sz, c_sz, c_sz, c_i]),
    "ksq_w4a16_packed_zeros_bytes": (c_sz, [c_sz, c_sz, c_sz, c_sz]),
    "ksq_w4a16_repack": (c_i, [c_p, c_i, c_p, c_sz, c_sz, c_sz, c_p]),
    "ksq_w4a16_unpack": (c_i, [c_p, c_i, c_p, c_sz, c_sz, c_sz, c_p]),
    "ksq_w4a16_repack_scales": (c_i, [c_p, c_i, c_p, c_sz, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_w4a16_unpack_scales": (c_i, [c_p, c_i, c_p, c_sz, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_w4a16_repack_zeros": (c_i, [c_p, c_i, c_p, c_sz, c_sz, c_sz, c_p]),
    "ksq_w4a16_unpack_zeros": (c_i, [c_p, c_i, c_p, c_sz, c_sz, c_sz, c_p]),
    "ksq_w4a16_workspace_size": (c_sz, [c_sz, c_sz, c_sz, c_sz, c_i]),
    "ksq_w4a16_gemm": (c_i, [c_p, c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_w4a16_gemm_f32": (c_i, [c_p, c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_w4a16_static_workspace_bytes": (c_sz, []),
    "ksq_w4a16_gemm_static": (c_i, [c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_fp8_group_quant": (c_i, [c_p, c_p, c_p, c_sz, c_sz, c_sz, c_i, c_i, c_i, c_p]),
    "ksq_fp8_blockwise_workspace_size": (c_sz, [c_sz, c_sz, c_sz]),
    "ksq_fp8_blockwise_gemm": (c_i, [c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_i, c_p, c_sz, c_p]),
    "ksq_fp8_blockwise_gemm_f32": (c_i, [c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_p, c_sz, c_p]),
    "ksq_moe_align_capacity": (c_sz, [c_sz, c_sz, c_sz]),
    "ksq_moe_align_scratch_bytes": (c_sz, [c_sz, c_sz]),
    "ksq_moe_align": (c_i, [c_p, c_sz, c_sz, c_sz, c_p, c_p, c_p, c_p, c_p]),
    "ksq_moe_w4a16_gemm": (c_i, [c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_sz, c_sz,
                                 c_sz, c_i, c_p]),
    "ksq_moe_w4a16_gate_up_silu": (c_i, [c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_sz, c_sz, c_sz,
                                         c_i, c_p]),
    "ksq_moe_w4a16_down_sum": (c_i, [c_p, c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_w4a16_repack_act_order": (c_i, [c_p, c_p, c_p, c_sz, c_sz, c_p]),
    "ksq_permute_columns": (c_i, [c_p, c_p, c_p, c_sz, c_sz, c_i, c_p]),
    "ksq_w4a16_repack_rows": (c_i, [c_p, c_p, c_p, c_sz, c_sz, c_sz, c_p]),
    "ksq_gather_columns": (c_i, [c_p, c_p, c_p, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_moe_permute_columns": (c_i, [c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_fp8_repack_weight": (c_i, [c_p, c_p, c_sz, c_sz, c_sz, c_p]),
    "ksq_fp8_unpack_weight": (c_i, [c_p, c_p, c_sz, c_sz, c_sz, c_p]),
    "ksq_fp8_channel_quant": (c_i, [c_p, c_p, c_p, c_sz, c_sz, c_i, c_i, c_p]),
    "ksq_fp8_tensor_gemm_workspace_size": (c_sz, [c_sz, c_sz, c_sz]),
    "ksq_fp8_tensor_gemm": (c_i, [c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_i, c_p, c_sz, c_p]),
    "ksq_moe_block_m": (c_sz, [c_sz, c_sz]),
    "ksq_moe_fp8_block_m": (c_sz, [c_sz, c_sz]),
    "ksq_moe_fp8_blockwise_gemm": (c_i, [c_p, c_p, c_p, c_i, c_sz, c_p, c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz,
                                         c_sz, c_sz, c_i, c_p]),
    "ksq_moe_fp8_down_sum": (c_i, [c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_moe_topk_softmax": (c_i, [c_p, c_p, c_p, c_sz, c_sz, c_sz, c_i, ctypes.c_float, c_i, c_p]),
    "ksq_moe_grouped_topk": (c_i, [c_p, c_p, c_p, c_p, c_sz, c_sz, c_sz, c_sz, c_sz, c_i, c_i, ctypes.c_float, c_i, c_p]),
    "ksq_moe_silu_mul": (c_i, [c_p, c_p, c_sz, c_sz, c_i, c_p]),
    "ksq_moe_sum": (c_i, [c_p, c_p, c_sz, c_sz, c_sz, c_i, c_p]),
    "ksq_w4a8_packed_weight_bytes": (c_sz, [c_sz, c_sz]),
    "ksq_w4a8_repack_weight": (c_i, [c_p, c_p, c_sz, c_sz, c_p]),
    "ksq_w4a8_unpack_weight": (c_i, [c_p, c_p, c_sz, c_sz, c_p]),
    "ksq_w4a8_static_quant": (c_i, [c_p, c_p, c_p, c_p, c_sz, c_sz, c_i, c_i, c_p]),
    "ksq_w4a8_workspace_size": (c_sz, [c_sz, c_sz, c_sz]),
    "ksq_w4a8_gemm": (c_i, [c_p, c_p, c_p, c_p, ctypes.c_float, c_p, c_sz, c_sz, c_sz, c_sz, c_i, c_p, c_sz, c_p]),
    "ksq_select_tile": (c_i, [c_i, c_sz, c_sz, c_sz, c_i, ctypes.POINTER(TileDesc)]),
    "ksq_set_small_problem_rule": (c_i, [c_i]),
    "ksq_diag_mfma_stream": (c_i, [c_i, c_i, c_i, c_p, c_p]),
    "ksq_diag_mfma_stream_flops": (ctypes.c_double, [c_i, c_i]),
}

_lib = None


class KsqError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("ksq status %d: %s" % (code, message))
        self.code = code


def load():
    """Load the built library; raises if it is missing (there is no fallback path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libksq_hip.so is not built: run `python -m ksanallm_amd.build` (needs hipcc)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise KsqError(rc, load().ksq_last_error_string().decode())


def set_small_problem_rule(enabled):
    """Process-wide: whether small problems of more than 32 rows run the decode-form kernels (default) or, like every
    larger one, the tile kernels.  Returns the previous setting."""
    return bool(load().ksq_set_small_problem_rule(1 if enabled else 0))


def select_tile(kind, m, n, k, dtype):
    d = TileDesc()
    check(load().ksq_select_tile(kind, m, n, k, dtype, ctypes.byref(d)))
    return {n: getattr(d, n) for n, _ in TileDesc._fields_}
