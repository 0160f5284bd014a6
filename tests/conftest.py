import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import ksq_oracle

    ksq_oracle.build()
    return ksq_oracle


@pytest.fixture
def tile_kernels():
    """Every problem of more than 32 rows runs the MFMA tile kernel for the length of the test: the library's rule that
    sends small ones (the sizes a CPU reference multiplies in seconds) to the decode-form kernels is switched off."""
    from ksanallm_amd import lib as L

    before = L.set_small_problem_rule(False)
    yield
    L.set_small_problem_rule(before)


@pytest.fixture(params=[True, False], ids=["small-problem-rule", "tile-kernels"])
def both_regimes(request):
    """The test runs twice: as the library decides by default, and with every problem of more than 32 rows on the tile
    kernels."""
    from ksanallm_amd import lib as L

    before = L.set_small_problem_rule(request.param)
    yield request.param
    L.set_small_problem_rule(before)
