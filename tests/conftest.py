import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "optimus-lm_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_lib():
    from oracle import clib
    clib.lib()
    return clib


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    from optimus import _native
    _native.lib()  # fail loudly if the HIP library is not built
    return torch.device("cuda:0")


def pytest_sessionfinish(session, exitstatus):
    """OM_PARITY_REPORT=<file>: append the measured parity margins (mean_rel, its bf16 floor and their
    ratio for every assert_bf16_parity call) so the bars in the tests can be kept near the figures."""
    path = os.environ.get("OM_PARITY_REPORT")
    if path:
        import util
        util.dump_parity_log(path)
