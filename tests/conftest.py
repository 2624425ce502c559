import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")


@pytest.fixture(scope="session")
def hip_device():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("a test marked gpu ran without a HIP device")
    return torch.device("cuda:0")


@pytest.fixture
def quant_settings():
    """``sage_ops.configure`` for one test: the process-wide settings of the one-read quantizers are put back (and the
    one-read kernels re-armed) when the test ends."""
    from ksanadit_amd import sage_ops

    before = sage_ops.one_read_state()
    yield sage_ops.configure
    sage_ops.configure(one_read=("k" if before["k"] else "") + ("v" if before["v"] else ""), wait_ticks=before["wait_ticks"])
