"""CPU-only checks of the C-ABI library and of the host-side logic around it:
the library loads, exports every function include/dlgrad_hip.h declares, reports errors
the way the boundary promises, compiles kernels for gfx950 without a GPU, and the
shape/stride helpers the launchers rely on behave."""
import ctypes
import os
import re

import numpy as np
import pytest

from dlgrad_amd import ffi, helpers
from dlgrad_amd.buffer import Buffer
from dlgrad_amd.codegen import hip_kernel as K
from dlgrad_amd.codegen import manifest
from dlgrad_amd.device import Device
from dlgrad_amd.dispatch import dispatcher
from dlgrad_amd.helpers import BinaryOps, BufferOps, CustomOps, UnaryOps
from dlgrad_amd.runtime import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "dlgrad_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dlg_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 25
    lib = ctypes.CDLL(ffi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
    assert sorted(ffi.EXPORTS) == names, "the Python binding table and the header disagree"


def test_calls_before_init_fail_with_a_message():
    lib = ffi.get_lib()
    if hip.available():
        pytest.skip("a GPU is present; the no-device error path is not reachable")
    with pytest.raises(ffi.HipError, match="no HIP device"):
        lib.init(0)
    with pytest.raises(MemoryError):
        lib.alloc(1024)
    with pytest.raises(ffi.HipError, match="dlg_hip_init"):
        lib.sync()
    assert lib.device_count() == 0
    with pytest.raises(ffi.HipError):
        Buffer.from_numpy(np.zeros((2, 2), np.float32), Device.HIP)     # loud, no CPU fallback


def test_hiprtc_compiles_for_gfx950_without_a_gpu_and_reports_errors():
    lib = ffi.get_lib()
    src, name, fmt = K.map_kernel("add", K.BINARY_EXPR["add"], ("vec", "row"), 4)
    code = lib.compile(src, name, list(K.COMPILE_OPTIONS))
    assert code[:4] == b"\x7fELF" and name.encode() in code
    assert fmt == "@PPPII"
    with pytest.raises(RuntimeError, match="Compilation failed"):
        lib.compile('extern "C" __global__ void broken() { this is not C++; }', "broken", list(K.COMPILE_OPTIONS))


def test_every_manifest_kernel_has_source_and_argument_format():
    import struct
    entries = manifest.load()
    assert len(entries) > 50
    for gen, params in entries:
        src, name, fmt = getattr(K, gen)(*params)
        assert f"void {name}(" in src
        assert struct.calcsize(fmt) > 0


def test_hip_runtime_registers_the_whole_operator_table():
    want = {BufferOps.CREATE, BufferOps.UNIFORM, BufferOps.ARANGE, BufferOps.FULL,
            BinaryOps.ADD, BinaryOps.SUB, BinaryOps.MUL, BinaryOps.DIV, BinaryOps.MATMUL, BinaryOps.GT,
            BinaryOps.GTE, BinaryOps.EQT, BinaryOps.CMP,
            UnaryOps.SUM, UnaryOps.MAX, UnaryOps.MEAN, UnaryOps.NEG, UnaryOps.EXP, UnaryOps.LOG, UnaryOps.POW,
            UnaryOps.SQRT, UnaryOps.RSQRT, UnaryOps.RELU, UnaryOps.ARGMAX, UnaryOps.WHERE, UnaryOps.CLAMP,
            UnaryOps.MASKED_FILL, UnaryOps.PERMUTE,
            CustomOps.CE_FORWARD, CustomOps.CE_BACKWARD, CustomOps.PRINT, CustomOps.EMBEDDING,
            CustomOps.TO_HOST, CustomOps.SOFTMAX, CustomOps.LOG_SOFTMAX}
    assert want <= dispatcher.registered(Device.HIP)
    with pytest.raises(KeyError):
        dispatcher.dispatch(UnaryOps.EXP, Device.METAL, x=None)


def test_device_names():
    assert Device.from_str("hip") is Device.HIP and Device.from_str("CPU") is Device.CPU
    assert Device.from_str("tpu") is None


def test_shape_helpers():
    assert helpers.calculate_stride((2, 3, 4)) == (12, 4, 1) and helpers.calculate_stride(()) == ()
    assert helpers.broadcast_shapes_2((3, 1), (3, 4)) == (3, 4)
    assert helpers.broadcast_shapes_2((4,), (2, 3, 4)) == (2, 3, 4)
    with pytest.raises(ValueError):
        helpers.broadcast_shapes_2((3, 2), (3, 4))
    assert helpers.get_broadcast_strides_2((2, 3, 4), (3, 1), (1, 1)) == (0, 1, 0)
    assert helpers.broadcast_shapes((5, 7), (4, 7, 3)) == ((1, 5, 7), (4, 7, 3), (4, 5, 3))
    with pytest.raises(ValueError):
        helpers.broadcast_shapes((5, 7), (6, 3))
    assert helpers.cal_sum_max_out_shape(3, 1, (2, 3, 4)) == (2, 4)
    assert helpers.cal_sum_max_out_shape(3, 1, (2, 3, 4), keepdim=True) == (2, 1, 4)
    assert helpers.cal_sum_max_out_shape(3, -1, (2, 3, 4)) == ()
    with pytest.raises(AssertionError):
        helpers.check_broadcast((2, 3), (4, 3))


def test_collapse_dims_finds_the_row_and_column_broadcast_patterns():
    cd, st = helpers.collapse_dims, helpers.calculate_stride
    # (16,4,128,128) * (16,4,128,1): rows of 128 with one value per row
    out = (16, 4, 128, 128)
    shape, (o, y) = cd(out, st(out), helpers.get_broadcast_strides_2(out, (16, 4, 128, 1), st((16, 4, 128, 1))))
    assert shape == (8192, 128) and o == (128, 1) and y == (1, 0)
    # (16,128,128) + (1,128,128): one "row" of 16384 repeated 16 times
    out = (16, 128, 128)
    shape, (o, y) = cd(out, st(out), helpers.get_broadcast_strides_2(out, (1, 128, 128), st((1, 128, 128))))
    assert shape == (16, 16384) and y == (0, 1)
    # same shapes collapse to one dim; a single value has all-zero strides
    shape, (o, y) = cd((4, 5), (5, 1), (5, 1))
    assert shape == (20,) and y == (1,)
    shape, (o, y) = cd((4, 5), (5, 1), (0, 0))
    assert shape == (20,) and y == (0,)
    # an interleaved pattern stays multi-dimensional
    shape, _ = cd((2, 3, 4, 5), st((2, 3, 4, 5)), (4, 0, 1, 0))
    assert len(shape) == 4


def test_device_pointer_views_keep_their_base_and_check_bounds():
    owner = hip.DevicePtr(0, 0)                     # address 0: nothing to free
    base = hip.DevicePtr(0x1000, 64, owner)         # a made-up address as a view, so nothing is freed for it either
    v = base + 4
    assert v.addr == 0x1010 and v.nbytes == 48 and v.base is owner and base.base is owner and owner.base is None
    with pytest.raises(IndexError):
        base + 17
    with pytest.raises(IndexError):
        base + -1
    assert "view" in repr(v) and "0x1010" in repr(v)


def test_pow_expression_is_repeated_multiplication():
    assert K.pow_expr(2) == "(x0 * x0)" or K.pow_expr(2) == "x0 * x0" or "x0" in K.pow_expr(2)
    x0 = 1.7

    def ev(n):
        return eval(K.pow_expr(n).replace("1.0f", "1.0").replace("powf", "pow"), {"x0": x0})
    for n in (0, 1, 2, 3, 5, 8, -1, -2):
        assert abs(ev(n) - x0 ** n) < 1e-12


# ---- failure handling on a device: every condition is forced from the host, every kernel exits normally
@pytest.mark.gpu
def test_failures_surface_as_python_exceptions_and_leave_the_device_usable():
    """The error contract of dlgrad/runtime/cpu.py:104,132,189 (MemoryError on a failed
    allocation) and :61-62 (RuntimeError on a failed compile), plus the host-side checks that
    stop a bad launch before it reaches the GPU."""
    from dlgrad_amd.runtime import hip
    if not hip.available():
        pytest.skip("no HIP device")
    import numpy as np
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    lib = hip.lib()
    in_use0, _, _ = lib.pool_stats()
    with pytest.raises(MemoryError, match="Failed to allocate"):
        hip.alloc(80 * 2 ** 30)                                   # 320 GiB of fp32 on a 288 GB card
    assert lib.pool_stats()[0] == in_use0                         # nothing is left registered by the failure
    with pytest.raises(RuntimeError, match="Compilation failed"):
        hip.code_object('extern "C" __global__ void broken(float* p) { p[0] = undefined_name; }', "broken")
    k = hip.kernel(K.map_kernel, "copy", "x0", ("vec",), 4)
    with pytest.raises(RuntimeError, match="empty grid"):
        hip.launch(k, 0, 256, 0, 0, 0, 1)
    with pytest.raises(RuntimeError, match="1024"):
        hip.launch(k, 1, 2048, 0, 0, 0, 1)
    with pytest.raises(RuntimeError, match="bad kernel handle"):
        hip.launch((10 ** 9, k[1]), 1, 64, 0, 0, 0, 1)
    with pytest.raises(ValueError, match="needs"):
        Buffer(hip.alloc(16), (5, 5), Device.HIP)                 # a view larger than its block
    with pytest.raises(ValueError, match="32-bit"):
        Buffer.uniform((2 ** 16, 2 ** 16), Device.HIP, "float32")
    x = Buffer.from_numpy(np.arange(12, dtype=np.float32).reshape(3, 4), Device.HIP)
    np.testing.assert_array_equal((x + x).numpy(), 2 * np.arange(12, dtype=np.float32).reshape(3, 4))


@pytest.mark.gpu
def test_capture_refuses_what_a_graph_cannot_replay():
    from dlgrad_amd.runtime import hip
    if not hip.available():
        pytest.skip("no HIP device")
    import numpy as np
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    lib = hip.lib()
    x = Buffer.from_numpy(np.ones((8, 8), np.float32), Device.HIP)
    g = hip.Graph()
    with g.arena():
        y = x + x
    in_use = lib.pool_stats()[0]
    with pytest.raises(RuntimeError):
        with g.capture():
            y = x + x
            y.numpy()                                             # a download inside a capture
    assert not hip.capturing()                                    # the failed capture was closed
    with pytest.raises(RuntimeError, match="replay the same numbers"):
        with g.capture():
            Buffer.uniform((4,), Device.HIP, "float32")
    assert not hip.capturing()
    with g.capture():
        y = x + x
    g.replay()
    np.testing.assert_array_equal(y.numpy(), np.full((8, 8), 2, np.float32))
    g.close()
    del y
    assert lib.pool_stats()[0] <= in_use


@pytest.mark.gpu
def test_an_allocation_that_misses_the_arena_during_a_capture_is_refused_on_the_host():
    """Under stream capture the allocator never reaches hipMalloc (nor the stream wait of its retry):
    a capture whose body asks for a size that the warm-up pass did not leave in the arena ends with a
    RuntimeError raised by the host, the capture is abandoned, and the device goes on working."""
    from dlgrad_amd.runtime import hip
    if not hip.available():
        pytest.skip("no HIP device")
    lib = hip.lib()
    x = Buffer.from_numpy(np.ones((8, 8), np.float32), Device.HIP)
    big = Buffer.from_numpy(np.ones((300, 300), np.float32), Device.HIP)
    (big + big).numpy()                                           # its kernel is loaded before any capture
    g = hip.Graph()
    with g.arena():
        y = x + x                                                 # the warm-up uses one 256-byte block at a time
    allocs_warm = lib.pool_stats()[2]
    with g.capture():                                             # ... and a repeat of it finds its block although y is still held
        y_again = x + x
    assert lib.pool_stats()[2] == allocs_warm
    g.close()
    g = hip.Graph()
    with g.arena():
        y = x + x
    del y, y_again
    allocs = lib.pool_stats()[2]
    with pytest.raises(RuntimeError, match="missed the arena during a capture"):
        with g.capture():
            z = big + big                                         # 360 000 bytes: no such block in the arena
    assert not hip.capturing()
    assert lib.pool_stats()[2] == allocs                          # no device allocation was made
    with pytest.raises(RuntimeError, match="missed the arena during a capture"):
        with g.capture():
            y1 = x + x
            y2 = x + x
            y3 = x + x                                            # three blocks at once of a size the arena holds twice
    assert not hip.capturing()
    del y1, y2                                                    # (back to the arena)
    np.testing.assert_array_equal((big + big).numpy(), np.full((300, 300), 2, np.float32))   # ordinary work goes on
    with g.capture():                                             # and the same Graph can still capture what fits
        y = x + x
    g.replay()
    np.testing.assert_array_equal(y.numpy(), np.full((8, 8), 2, np.float32))
    g.close()


@pytest.mark.gpu
def test_pinned_staging_uploads_without_a_wait_and_inside_a_captured_graph():
    """A page-locked array is uploaded by an enqueued DMA; recorded into a graph, the copy
    re-reads the array on every replay, so a loop refills it between replays (after a sync)
    and nothing else crosses the host boundary."""
    from dlgrad_amd.runtime import hip
    if not hip.available():
        pytest.skip("no HIP device")
    lib = hip.lib()
    rng = np.random.default_rng(8)
    held = set(hip._pinned)                                       # (the runtime keeps a few small staging blocks of its own)
    stage = hip.pinned_empty((128, 784))
    assert stage.dtype == np.float32 and stage.shape == (128, 784) and hip._is_pinned(stage)
    stage[:] = rng.random((128, 784), dtype=np.float32)
    want = stage.copy()
    x = Buffer.from_numpy(stage, Device.HIP)                      # enqueued, not waited for
    np.testing.assert_array_equal(x.numpy(), want)                # numpy() waits for the stream
    with pytest.raises(RuntimeError, match="host_alloc block"):
        lib.h2d_async(x.ptr.addr, want.ctypes.data, want.nbytes)  # pageable memory is refused
    g = hip.Graph()
    with g.arena():
        y = x * 2.0
    with g.capture():
        x.upload_(stage)                                          # a memcpy node that reads `stage` at replay time
        y = x * 2.0
    for k in range(3):
        lib.sync()                                                # the previous replay has read the staging array
        stage[:] = np.float32(k + 1)
        g.replay()
        np.testing.assert_array_equal(y.numpy(), np.full((128, 784), 2 * (k + 1), np.float32))
    g.close()
    del stage, x, y
    import gc
    gc.collect()
    assert set(hip._pinned) == held                               # the page-locked block went back


def _run_bench(*args):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, DLGRAD_HIP_COMPILE_ONLY="1")
    return subprocess.run([sys.executable, os.path.join(root, "bench.py"), *args], capture_output=True, text=True,
                          env=env, cwd=root, timeout=600)


def test_bench_refuses_more_than_one_gpu_with_a_message():
    r = _run_bench("--gpus", "2")
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_bench_prints_one_json_line_with_the_contract_keys():
    """Compile-only mode runs the whole host side of a workload without a device (timings are
    placeholders): the line must parse and carry every key the harness reads."""
    import json
    r = _run_bench("--workload", "mlp", "--steps", "2", "--warmup", "1", "--no-cpu")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 2 and out["warmup"] == 1 and out["vs_baseline"] is None
    assert out["dtype"] == "f32" and out["data"] == "synthetic" and "workload" in out["config"]


@pytest.mark.gpu
def test_large_blocks_are_staggered_and_recycled_whole():
    """Allocations of 8 MiB and more start 4 KiB apart (mod 16 KiB) from one to the next, so that the
    operands of an element-wise kernel do not meet the same DRAM bank at the same moment; freeing returns
    the whole block (the next block of that size reuses it, whatever its offset), and contents written
    through an offset pointer read back intact up to the last byte asked for."""
    from dlgrad_amd.runtime import hip
    if not hip.available():
        pytest.skip("no HIP device")
    import numpy as np
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    lib = hip.lib()
    n = (8 << 20) // 4 + 1021                                     # just over 8 MiB, not a round size
    ptrs = [hip.alloc(n) for _ in range(5)]
    offs = [p.addr % (4 * 4096) for p in ptrs]
    assert all(p.addr % 4096 == 0 for p in ptrs)
    assert [(b - a) % (4 * 4096) for a, b in zip(offs, offs[1:])] == [4096] * 4, offs
    small = [hip.alloc(1024) for _ in range(3)]
    assert len({p.addr % 256 for p in small}) == 1                # small blocks are left alone
    in_use, cached, allocs = lib.pool_stats()
    del ptrs
    again = [hip.alloc(n) for _ in range(5)]
    assert lib.pool_stats()[2] == allocs, "freed large blocks were not reused"
    data = np.arange(n, dtype=np.float32)
    for p in again:
        b = Buffer(p, (n,), Device.HIP)
        b.upload_(data)
    for p in again:
        np.testing.assert_array_equal(Buffer(p, (n,), Device.HIP).numpy(), data)


def _run_pytest_subprocess(env_extra: dict):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = {k: v for k, v in os.environ.items() if k not in ("DLGRAD_HIP_COMPILE_ONLY", "DLGRAD_HIP_MANIFEST")}
    env.update(env_extra)
    return subprocess.run([sys.executable, "-m", "pytest", "tests/test_hip_elementwise.py", "-m", "gpu", "-q", "-x",
                           "-p", "no:cacheprovider", "-k", "test_fills"], capture_output=True, text=True, env=env,
                          cwd=root, timeout=600)


def test_a_stray_compile_only_variable_fails_the_gpu_tests_instead_of_passing_them():
    """Compile-only mode launches nothing and compares nothing; only the kernel-recording run
    (which also names a manifest file, on a machine without a device) may use it for the tests."""
    r = _run_pytest_subprocess({"DLGRAD_HIP_COMPILE_ONLY": "1"})
    assert r.returncode == 3 and "DLGRAD_HIP_COMPILE_ONLY" in (r.stdout + r.stderr), (r.returncode, r.stdout[-500:])


@pytest.mark.gpu
def test_reduce_full_checks_its_arguments_on_the_host():
    """dlg_hip_reduce_full launches twice on the caller's word; what the kernels and their grid assume
    (access width, alignment, element count, room for the partial results) is checked before."""
    from dlgrad_amd.runtime import hip
    if not hip.available():
        pytest.skip("no HIP device")
    import numpy as np
    from dlgrad_amd.codegen import hip_kernel as K
    from dlgrad_amd.ffi import HipError
    lib = hip.lib()
    k1, k4 = hip.kernel(K.reduce_full_kernel, "sum", 1)[0], hip.kernel(K.reduce_full_kernel, "sum", 4)[0]
    n = 100_000
    x, out, ws = hip.alloc(n + 1), hip.alloc(1), hip.alloc(64)
    ones = np.ones(n + 1, np.float32)                                           # kept alive across the copy
    lib.h2d(x.addr, ones.ctypes.data, 4 * (n + 1))
    G = ((n + 3) // 4 + 2047) // 2048
    lib.reduce_full(k4, k4, x.addr, n, 4, 1.0, out.addr, ws.addr, 4 * G)
    got = np.empty(1, np.float32)
    lib.d2h(got.ctypes.data, out.addr, 4)
    assert got[0] == n
    lib.reduce_full(k1, k4, x.addr + 4, n, 1, 2.0, out.addr, ws.addr, 256)      # unaligned input, 4-byte reads, a mean-like divisor
    lib.d2h(got.ctypes.data, out.addr, 4)
    assert got[0] == n / 2
    for args, msg in (((k4, k4, x.addr + 4, n, 4, 1.0, out.addr, ws.addr, 256), "aligned"),
                      ((k4, k4, x.addr, n, 3, 1.0, out.addr, ws.addr, 256), "vec"),
                      ((k4, k4, x.addr, 0, 4, 1.0, out.addr, ws.addr, 256), "n must"),
                      ((k4, k4, x.addr, n, 4, 1.0, out.addr, ws.addr, 4 * G - 4), "partial results need"),
                      ((k4, k4, x.addr, n, 4, 1.0, out.addr, 0, 0), "partial results need"),
                      ((k4, k4, x.addr, n, 4, 1.0, out.addr, ws.addr + 4, 256), "partial results need"),
                      ((k4, 10 ** 6, x.addr, n, 4, 1.0, out.addr, ws.addr, 256), "handle"),
                      ((k4, k4, x.addr, 2048 * 4 * 65536 + 1, 4, 1.0, out.addr, ws.addr, 256), "at most")):
        with pytest.raises(HipError, match=msg):
            lib.reduce_full(*args)
    lib.sync()


@pytest.mark.gpu
def test_event_and_graph_handles_are_checked():
    """Handles are indices into the library's own tables: a number it never gave out, or one that
    was destroyed, is refused with a message instead of being used as a pointer."""
    from dlgrad_amd.runtime import hip
    if not hip.available():
        pytest.skip("no HIP device")
    from dlgrad_amd.ffi import HipError
    lib = hip.lib()
    e0, e1 = lib.event_create(), lib.event_create()
    lib.event_record(e0)
    lib.event_record(e1)
    lib.event_sync(e1)
    assert lib.event_elapsed_ms(e0, e1) >= 0.0
    lib.event_destroy(e1)
    for bad in (e1, 0, 10 ** 9):
        with pytest.raises(HipError, match="bad event handle"):
            lib.event_record(bad)
        with pytest.raises(HipError, match="bad event handle"):
            lib.event_elapsed_ms(e0, bad)
    with pytest.raises(HipError, match="bad graph handle"):
        lib.graph_launch(10 ** 9)
    lib.event_destroy(e0)
    assert hip.props()["name"], "the device name must not be empty"


def test_tolerance_comparator_never_lets_a_lone_nan_or_infinity_pass():
    """The helper every floating-point parity test rests on: a NaN or infinity on one side only is an
    infinite error (np.testing.assert_allclose, the reference's comparator, behaves the same way);
    NaN against NaN and equal infinities are matches."""
    from tests.hip_util import check, rel_err
    nan, inf = float("nan"), float("inf")
    with pytest.raises(AssertionError):
        check(np.array([1, nan, 3], np.float32), np.array([1, 2, 3], np.float32), 1e-6)
    with pytest.raises(AssertionError):
        check(np.array([1, 2, 3], np.float32), np.array([1, nan, 3], np.float32), 1e-6)
    with pytest.raises(AssertionError):
        check(np.array([1, inf, 3], np.float32), np.array([1, 2, 3], np.float32), 1e-6)
    with pytest.raises(AssertionError):
        check(np.array([1, inf, 3], np.float32), np.array([1, -inf, 3], np.float32), 1e-6)
    with pytest.raises(AssertionError):
        check(np.array([1, 2.001, 3], np.float32), np.array([1, 2, 3], np.float32), 1e-6)
    assert rel_err(np.array([nan]), np.array([0.0])) == inf
    check(np.array([1, nan, inf, -inf, 0], np.float32), np.array([1, nan, inf, -inf, 0], np.float32), 1e-6)
    check(np.array([1, 2.0000001, 3], np.float32), np.array([1, 2, 3], np.float32), 1e-6)
    check(np.zeros((0,), np.float32), np.zeros((0,), np.float32), 1e-6)


def test_first_tile_timing_of_a_process_says_so_once(monkeypatch, tmp_path):
    """A product shape that is in no tile table is timed with every plausible tile on first use, which makes
    a user's first step many times slower: the first such timing of a process warns, naming the shape, the
    cost and the switch; later ones stay silent.  (Host logic only: launches and events are stand-ins.)"""
    import warnings
    from dlgrad_amd.runtime.hip import HIP

    class Events:
        def event_create(self): return 1
        def event_record(self, e): pass
        def event_sync(self, e): pass
        def event_elapsed_ms(self, a, b): return 1.0
        def event_destroy(self, e): pass

    monkeypatch.setattr(hip, "lib", lambda: Events())
    monkeypatch.setattr(hip, "COMPILE_ONLY", False)
    monkeypatch.setattr(HIP, "_launch_matmul", staticmethod(lambda *a, **k: None))
    monkeypatch.setattr(HIP, "_tile_candidates", staticmethod(lambda M, N, batch, Kd=0, split=False: ["128x128x32_w2x2"]))
    monkeypatch.setattr(HIP, "MATMUL_TUNED_FILE", str(tmp_path / "tuned.json"))
    monkeypatch.setattr(HIP, "_tuned_new", {})
    monkeypatch.setattr(HIP, "_tune_warned", False)
    table = dict(HIP._tuned_table())
    try:
        with pytest.warns(RuntimeWarning, match=r"1,3000,1000,2000.*DLGRAD_HIP_MATMUL_TUNE=0"):
            assert HIP._tune_tile("1,3000,1000,2000", True, True, 3000, 1000, 1, (0, 0, 0, 3000, 1000, 2000), False, False) == "128x128x32_w2x2"
        with warnings.catch_warnings():
            warnings.simplefilter("error")                                # a second shape: timed without a word
            assert HIP._tune_tile("1,3001,1000,2000", True, True, 3001, 1000, 1, (0, 0, 0, 3001, 1000, 2000), False, False) == "128x128x32_w2x2"
        import json
        assert set(json.load(open(tmp_path / "tuned.json"))) == {"1,3000,1000,2000", "1,3001,1000,2000"}
    finally:
        HIP._tuned_table().clear()
        HIP._tuned_table().update(table)


def test_tile_names_that_cut_k_are_parsed_and_planned_on_the_host():
    """Host logic of the product launcher: "base/s" cuts k into s slices across blocks (a workspace and a column-sum
    launch), "base*g" among g groups of wavefronts inside a block.  Every slice is a whole number of the tile's k
    steps and none is empty; groups all take the same number of steps, and a k of fewer steps than groups gets fewer
    groups, down to the plain tile.  Names that are no tile are refused (the tile tables are read through this)."""
    from dlgrad_amd.codegen import hip_kernel as K
    from dlgrad_amd.runtime.hip import HIP
    assert HIP._split_of("128x128/4") == ("128x128", 4) and HIP._groups_of("128x128/4") == 1
    assert HIP._split_of("64x64k32*4") == ("64x64k32", 1) and HIP._groups_of("64x64k32*4") == 4
    assert HIP._split_of("64x64") == ("64x64", 1) and HIP._groups_of("64x64") == 1
    for good in ("64x64", "256x128k32", "128x128/16", "64x64k64*2", "32x32*8", "32x32m16*4"):
        assert HIP._valid_tile(good), good
    for bad in ("65x64", "64x64/0", "64x64/x", "64x64*5", "64x64*x", "128x128/2*2", "256x256*2", "", "rows"):
        assert not HIP._valid_tile(bad), bad
    for tile, Kd in (("128x128/4", 4096), ("128x128/4", 1030), ("64x64k64/16", 2048), ("64x64m16/3", 700), ("128x64/2", 40)):
        slices, kchunk = HIP._split_plan(tile, Kd)
        bk = K.MATMUL_CONFIGS[HIP._split_of(tile)[0]][4]
        assert kchunk % bk == 0 and (slices - 1) * kchunk < Kd <= slices * kchunk and 1 <= slices <= HIP._split_of(tile)[1], (tile, Kd, slices, kchunk)
    for tile, Kd, want in (("64x64k64*2", 1024, 2), ("64x64k32*4", 96, 3), ("32x32*8", 40, 3), ("128x128*2", 20, 1), ("64x64*3", 4096, 3), ("32x32m16*4", 1030, 4)):
        groups, kchunk = HIP._group_plan(tile, Kd)
        bk = K.MATMUL_CONFIGS[HIP._split_of(tile)[0]][4]
        assert groups == want and kchunk % bk == 0 and groups * kchunk >= Kd, (tile, Kd, groups, kchunk)
    # what is offered for timing: split forms only for few-tile products with a long k, and every candidate is a valid tile
    few = HIP._tile_candidates(512, 512, 1, 2048, True)
    assert any("/" in t for t in few) and any("*" in t for t in few) and all(HIP._valid_tile(t) for t in few)
    assert not any("/" in t or "*" in t for t in HIP._tile_candidates(512, 512, 1, 2048, False))
    assert HIP._splitk_eligible(768, 768, 8192, 1) and not HIP._splitk_eligible(4096, 4096, 4096, 1) and not HIP._splitk_eligible(512, 512, 256, 1)
