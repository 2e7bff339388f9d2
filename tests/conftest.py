import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "scalable-flash-native-sparse-attention_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _tuning_values_do_not_leak():
    """nsa_set_tuning keeps process-wide overrides: whatever a test sets (or leaves set when it fails half way) is
    dropped before the next test runs."""
    yield
    try:
        from flash_nsa import _lib
        if _lib.LIB._dll is not None:
            _lib.call("nsa_reset_tuning")
    except ImportError:
        pass
