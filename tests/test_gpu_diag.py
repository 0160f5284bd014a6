"""ksq_diag_mfma_stream: the bare matrix-instruction streams bench.py --mfma-stream times."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_mfma_stream_runs_every_kind_and_checks_its_arguments():
    from ksanallm_amd import lib as L
    lib = L.load()
    sink = torch.zeros(256 * 512, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    for kind in range(6):
        for constant in (0, 1):
            L.check(lib.ksq_diag_mfma_stream(kind, constant, 8, sink.data_ptr(), stream))
        per_iter = lib.ksq_diag_mfma_stream_flops(kind, 1)
        assert per_iter == 256 * 8 * (2 ** 20 if kind in (2, 5) else 2 ** 19)
        assert lib.ksq_diag_mfma_stream_flops(kind, 10) == 10 * per_iter
    torch.cuda.synchronize()
    assert not sink.any()   # the sums of these operands never match the sentinel: nothing is written
    assert lib.ksq_diag_mfma_stream(6, 0, 8, sink.data_ptr(), stream) == 1
    assert lib.ksq_diag_mfma_stream(0, 0, 0, sink.data_ptr(), stream) == 1
    assert lib.ksq_diag_mfma_stream(0, 0, 8, None, stream) == 1
    assert lib.ksq_diag_mfma_stream_flops(9, 8) == 0.0
