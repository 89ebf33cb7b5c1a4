import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


@pytest.fixture(scope="session")
def rng_seed():
    return 1234


@pytest.fixture(autouse=True)
def default_switches(monkeypatch):
    """Every test starts from the documented defaults whatever the environment says (fused ops on,
    no forced tile); tests of the alternatives switch them with monkeypatch themselves."""
    from dlgrad_amd import ops
    monkeypatch.setattr(ops, "FUSED", True)
    try:
        from dlgrad_amd.runtime.hip import HIP
    except Exception:                 # the shared library is not built: CPU-only tests still run
        return
    monkeypatch.setattr(HIP, "MATMUL_FORCE", None)
    monkeypatch.setattr(HIP, "ROW_MATMUL", True)
    monkeypatch.setattr(HIP, "DECODE_FUSED", True)
