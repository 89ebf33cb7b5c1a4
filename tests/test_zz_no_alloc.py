"""The allocation-free full reduction (dlg_hip_reduce_full_static) against the entry point it is
a variant of (dlg_hip_reduce_full with a caller's workspace): same kernels, same launches, the
partial results in the library's static device array instead."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _setup():
    from dlgrad_amd.runtime import hip
    if not hip.available():
        pytest.skip("no HIP device")
    assert not hip.COMPILE_ONLY, "compile-only mode executes nothing"
    from dlgrad_amd.codegen import hip_kernel as K
    return hip, hip.lib(), K


def _both(hip, lib, K, op, x_dev, n, vec, divisor):
    """(result through the workspace entry point, result through the static one, device allocations made by the second)."""
    k_stage = hip.kernel(K.reduce_full_kernel, op, vec)[0]
    k_fold = hip.kernel(K.reduce_full_kernel, op, 4)[0]
    G = ((n + vec - 1) // vec + 2047) // 2048
    ws, out_a, out_b = hip.alloc(max(G, 1)), hip.alloc(1), hip.alloc(1)
    lib.reduce_full(k_stage, k_fold, x_dev, n, vec, divisor, out_a.addr, ws.addr, 4 * G)
    before = lib.pool_stats()
    lib.reduce_full_static(k_stage, k_fold, x_dev, n, vec, divisor, out_b.addr)
    after = lib.pool_stats()
    a, b = np.empty(1, np.float32), np.empty(1, np.float32)
    lib.d2h(a.ctypes.data, out_a.addr, 4)
    lib.d2h(b.ctypes.data, out_b.addr, 4)
    return a[0], b[0], (after[0] - before[0], after[2] - before[2])


def test_static_scratch_reduction_equals_the_workspace_one_twice_in_a_row():
    hip, lib, K = _setup()
    rng = np.random.default_rng(77)
    big, small = 40_000_003, 70_001                      # 4883 partials, then 9: the second call leaves most of the array stale
    host = rng.standard_normal(big).astype(np.float32)
    x = hip.alloc(big)
    lib.h2d(x.addr, host.ctypes.data, 4 * big)
    for op in ("sum", "max"):
        for n in (big, small):                           # two calls in a row on the same array, the second smaller
            a, b, grew = _both(hip, lib, K, op, x.addr, n, 4, 1.0)
            assert a.tobytes() == b.tobytes(), (op, n, a, b)
            assert grew == (0, 0), "the static entry point went to the allocator"
            want = host[:n].astype(np.float64).sum() if op == "sum" else host[:n].max()
            assert abs(float(b) - want) <= 1e-5 * max(1.0, abs(want)) + (1e-3 if op == "sum" else 0), (op, n, b, want)
    a, b, _ = _both(hip, lib, K, "sum", x.addr + 4, small, 1, float(small))        # unaligned view, 4-byte reads, a mean
    assert a.tobytes() == b.tobytes()
    a, b, _ = _both(hip, lib, K, "max", x.addr, 5, 4, 1.0)                          # one block: no partials at all
    assert a.tobytes() == b.tobytes() and b == host[:5].max()


def test_static_scratch_reduction_refuses_what_does_not_fit():
    hip, lib, K = _setup()
    from dlgrad_amd.ffi import HipError
    k = hip.kernel(K.reduce_full_kernel, "sum", 4)[0]
    x, out = hip.alloc(1024), hip.alloc(1)
    with pytest.raises(HipError, match="at most 65536"):
        lib.reduce_full_static(k, k, x.addr, 2048 * 4 * 65536 + 1, 4, 1.0, out.addr)
    with pytest.raises(HipError, match="vec"):
        lib.reduce_full_static(k, k, x.addr, 1024, 2, 1.0, out.addr)
    lib.sync()
