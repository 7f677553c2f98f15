import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True, scope="session")
def _kernels_at_first_use_off():
    """Compilation at first use is on for users; the suite keeps it off (the table-driven kernels stay covered and dozens
    of small descriptors are not compiled), ``tests/test_jit.py`` switches it on for its cases; ``CUEQ_AMD_TEST_JIT=1`` leaves it on for the whole run."""
    from cuequivariance_amd import jit

    if os.environ.get("CUEQ_AMD_TEST_JIT", "0") == "1":  # the whole suite on the kernels compiled at first use
        yield
        return
    jit.enable(False)
    yield



@pytest.fixture
def jit_on(tmp_path, monkeypatch):
    """Compilation at first use switched on for one test, into an empty cache; the previous state comes back afterwards."""
    from cuequivariance_amd import jit

    was = jit.enabled()
    monkeypatch.setenv("CUEQ_AMD_JIT_CACHE", str(tmp_path))
    jit.enable(True)
    yield
    jit.enable(was)
