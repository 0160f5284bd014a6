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


@pytest.fixture(autouse=True)
def _small_problem_rule_restored():
    """Whatever a test did with the library's process-wide small-problem rule (helpers.each_regime), the next test
    starts from the default."""
    yield
    from ksanallm_amd import lib as L

    if L._lib is not None:
        L.set_small_problem_rule(True)
