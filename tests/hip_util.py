"""Shared helpers of the GPU parity tests."""
import numpy as np
import pytest

from dlgrad_amd.buffer import Buffer
from dlgrad_amd.device import Device
from dlgrad_amd.runtime import hip


def require_gpu():
    """Skips where there is no device.  Compile-only mode (the kernel-recording run, admitted by
    conftest only without a device and with DLGRAD_HIP_MANIFEST set) goes through the host side
    of the test so that the kernels it asks for are listed; it executes and compares nothing."""
    if not (hip.available() or hip.COMPILE_ONLY):
        pytest.skip("no HIP device")
    assert not (hip.COMPILE_ONLY and hip.available()), "compile-only mode with a device present tests nothing"


def dev(a) -> Buffer:
    return Buffer.from_numpy(np.ascontiguousarray(a, dtype=np.float32), Device.HIP)


def rel_err(got, want) -> float:
    """max |got-want| / max(|want|, tiny) over elements.  Exact matches (incl. equal infinities and
    NaN on both sides) count 0; a NaN on one side only, or an infinity against anything else, is an
    infinite error -- as with np.testing.assert_allclose, a lone NaN can never pass a tolerance."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    same = (got == want) | (np.isnan(got) & np.isnan(want))
    with np.errstate(all="ignore"):
        e = np.abs(got - want) / np.maximum(np.abs(want), 1e-30)
    e = np.where(same, 0.0, np.where(np.isfinite(e), e, np.inf))
    return float(np.max(e)) if e.size else 0.0


def check(got, want, tol: float, what: str = "") -> None:
    if hip.COMPILE_ONLY:                     # the recording run: nothing was computed
        return
    got = np.asarray(got)
    assert got.shape == np.asarray(want).shape, f"{what}: shape {got.shape} vs {np.asarray(want).shape}"
    if tol == 0:
        np.testing.assert_array_equal(got, want, err_msg=what)
    else:
        e = rel_err(got, want)
        assert e <= tol, f"{what}: relative error {e:.3e} > {tol:.1e}"
