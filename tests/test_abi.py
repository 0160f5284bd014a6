"""The C-ABI library loads on a machine without a GPU and exports exactly what include/ksq.h declares."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ksq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ksq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from ksanallm_amd import lib as L
    lib = L.load()
    names = declared_functions()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(L.SIGNATURES) == names
    assert lib.ksq_version() == 1
    assert lib.ksq_last_error_string() is not None


def test_size_queries_and_tile_selection_are_host_only():
    from ksanallm_amd import lib as L
    lib = L.load()
    assert lib.ksq_w4a16_packed_weight_bytes(1, 4096, 4096) == 4096 * 4096 // 2
    assert lib.ksq_w4a16_packed_scales_bytes(1, 4096, 4096, 128, L.F16) == 32 * 4096 * 2
    assert lib.ksq_w4a16_packed_zeros_bytes(1, 4096, 14336, 128) == 32 * 14336
    assert lib.ksq_moe_align_capacity(64, 256, 16) == 64 + 256 * 15
    d = L.select_tile(L.KIND_W4A16, 1, 4096, 4096, L.F16)
    assert d["kernel"] == 0 and d["grid"] >= 256
    # deterministic: same answer every time, no timing involved
    assert d == L.select_tile(L.KIND_W4A16, 1, 4096, 4096, L.F16)
    import pytest
    with pytest.raises(L.KsqError):
        L.select_tile(99, 1, 16, 128, 0)
    # W4A8: packed size, and a workspace that covers every token count up to the maximum it was asked for
    assert lib.ksq_w4a8_packed_weight_bytes(5120, 5120) == 5120 * 5120 // 2
    assert lib.ksq_w4a8_workspace_size(32, 5120, 5120) == 0        # the streaming kernel needs none
    need = lib.ksq_w4a8_workspace_size(4096, 256, 8192)
    assert need > 0
    for m in (33, 64, 100, 128, 129, 700, 4096):
        assert lib.ksq_w4a8_workspace_size(m, 256, 8192) <= need
    assert lib.ksq_w4a8_workspace_size(64, 256, 100) == 0          # k not a multiple of 128: no kernel, no scratch


def test_small_problem_rule_and_its_switch():
    """Above 32 rows the tile kernels, but for small problems; the switch sends those to the tile kernels too, the
    descriptor follows it, and the workspace query covers both settings."""
    from ksanallm_amd import lib as L
    lib = L.load()
    small, large = (128, 4096, 4096), (160, 14336, 4096)  # ceil(m/32) * n * k = 2^26 and 5 * 14336 * 4096 > 2^28
    assert L.select_tile(L.KIND_W4A16, *small, L.BF16)["kernel"] == 0
    assert L.select_tile(L.KIND_W4A16, *large, L.BF16)["kernel"] == 1
    assert L.select_tile(L.KIND_W4A16, 513, 256, 256, L.BF16)["kernel"] == 1      # never beyond 512 rows
    assert L.select_tile(L.KIND_W4A16, 64, 25600, 5120, L.F16)["kernel"] == 0      # 2 * n * k < 2^28
    assert L.select_tile(L.KIND_W4A16, 64, 5120, 25600, L.F16)["kernel"] == 1      # K the long side by 4x: 2^27
    assert L.select_tile(L.KIND_FP8_BLOCKWISE, 64, 4608, 7168, L.BF16)["kernel"] == 0
    assert L.select_tile(L.KIND_FP8_BLOCKWISE, 64, 24576, 1536, L.BF16)["kernel"] == 1  # n > 4 k
    assert L.select_tile(L.KIND_FP8_BLOCKWISE, 96, 7168, 7168, L.BF16)["kernel"] == 1   # 3 * n * k > 5 * 2^24
    assert L.select_tile(L.KIND_FP8_BLOCKWISE, 128, 4096, 4096, L.BF16)["kernel"] == 0
    assert L.select_tile(L.KIND_FP8_BLOCKWISE, 64, 7168, 7168, L.BF16)["kernel"] == 1
    assert L.select_tile(L.KIND_W4A8, 96, 5120, 5120, L.BF16)["kernel"] == 0
    assert L.select_tile(L.KIND_W4A8, 256, 5120, 5120, L.BF16)["kernel"] == 1
    ws_on = lib.ksq_w4a16_workspace_size(128, 4096, 14336, 128, L.BF16)
    assert L.set_small_problem_rule(False) is True
    try:
        assert L.select_tile(L.KIND_W4A16, *small, L.BF16)["kernel"] == 1
        assert L.select_tile(L.KIND_FP8_BLOCKWISE, 128, 4096, 4096, L.BF16)["kernel"] == 1
        assert L.select_tile(L.KIND_W4A8, 96, 5120, 5120, L.BF16)["kernel"] == 1
        d = L.select_tile(L.KIND_W4A16, 128, 4096, 14336, L.BF16)
        assert d["kernel"] == 1 and d["split_k"] > 1
        assert lib.ksq_w4a16_workspace_size(128, 4096, 14336, 128, L.BF16) == ws_on >= d["split_k"] * 128 * 4096 * 4
    finally:
        assert L.set_small_problem_rule(True) is False
    assert L.select_tile(L.KIND_W4A16, *small, L.BF16)["kernel"] == 0
