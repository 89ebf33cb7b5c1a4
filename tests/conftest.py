import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


def compile_only_refusal() -> str:
    """Why this test session must not run in compile-only mode, or "" if it may.

    DLGRAD_HIP_COMPILE_ONLY=1 skips every launch and every comparison, so a GPU test "passes"
    there without having executed a kernel.  The one legitimate use is the run that records
    which kernels the tests ask for (dlgrad_amd.codegen.manifest --record), which sets
    DLGRAD_HIP_MANIFEST as well and runs where there is no device.  Anything else -- the
    variable inherited by accident, or set on a machine that has a GPU -- ends the session
    with an error instead of a green result."""
    if os.environ.get("DLGRAD_HIP_COMPILE_ONLY") != "1":
        return ""
    if not os.environ.get("DLGRAD_HIP_MANIFEST"):
        return ("DLGRAD_HIP_COMPILE_ONLY=1 is set without DLGRAD_HIP_MANIFEST: in that mode no kernel runs and no "
                "result is compared, so the GPU tests would pass without testing anything; unset it")
    try:
        from dlgrad_amd.runtime import hip
        has_device = hip.available()
    except Exception:
        has_device = False
    if has_device:
        return ("DLGRAD_HIP_COMPILE_ONLY=1 on a machine with a HIP device: the tests would pass without executing "
                "a kernel; unset it (a run with DLGRAD_HIP_MANIFEST alone records the kernels while really running)")
    return ""


def pytest_sessionstart(session):
    why = compile_only_refusal()
    if why:
        pytest.exit(why, returncode=3)


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
    # Tiles come from the committed table and the model, not from timings taken on this machine: which tile wins a
    # timing differs from machine to machine, and among the candidates of a few-tile product are the forms that cut k
    # into slices, which change result bits -- a test that compares two routes bit for bit must not depend on that.
    # The tests of the timing itself switch it on.
    monkeypatch.setattr(HIP, "MATMUL_TUNE", False)
