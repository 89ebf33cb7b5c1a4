"""The `hip` runtime: one static method per (op, Device.HIP) pair of the dispatch table.

Plays the part dlgrad/runtime/cpu.py:43-1061 plays for the CPU: allocate the
output, pick the kernel for the ranks/shapes at hand, pack its arguments, call
it, return the bare pointer.  The differences are the MI355X ones:

* kernels are HIP sources from `dlgrad_amd.codegen.hip_kernel`, compiled for
  gfx950 by hiprtc through libdlgrad_hip.so and cached as code objects on disk
  (the reference caches .so files per source hash, cpu.py:64-78, and stats the
  file on every call, cpu.py:268; here the handle lookup is an in-process dict);
* outputs come from a pooled device allocator and are returned to it by the
  `DevicePtr` finaliser (the reference uses ffi.gc(ptr, free_ptr), cpu.py:102);
* launches are asynchronous on one stream; only `TO_HOST` waits;
* Python floats arrive by value, never through memory.

Nothing here falls back to another device: a missing library or GPU raises.
"""
from __future__ import annotations

import hashlib
import json
import math
import os
import struct
import warnings

import numpy as np

from dlgrad_amd import ffi as _ffi
from dlgrad_amd.buffer import Buffer, HostScalar
from dlgrad_amd.codegen import hip_kernel as K
from dlgrad_amd.device import Device
from dlgrad_amd.dispatch import dispatcher
from dlgrad_amd.helpers import (
    CACHE_DIR,
    STRICT_REFERENCE,
    BinaryOps,
    BufferOps,
    CustomOps,
    UnaryOps,
    broadcast_shapes_2,
    calculate_stride,
    collapse_dims,
    get_broadcast_strides_2,
    prod_,
)

_state = {"lib": None, "ready": False, "props": None}
_handles: dict = {}            # (generator, params) -> (kernel handle, struct.Struct)
kernel_names: dict = {}        # id of such a pair -> the kernel's name in its code object (what a profiler shows)
launch_count = 0               # launches issued since import (read by the benchmarks)

# Ahead-of-time mode for the build step: no device is touched, every kernel a workload
# asks for is compiled into the on-disk cache and listed, launches are skipped and
# results are meaningless.  It exists so a machine without a GPU can compile exactly the
# code objects a later GPU run will load; it is never a way to compute anything.
COMPILE_ONLY = os.environ.get("DLGRAD_HIP_COMPILE_ONLY") == "1"
requested_kernels: set = set()  # (generator name, params) seen by kernel()
compiled_now: list = []         # kernels that missed the on-disk cache in this process


class _CompileOnlyLib:
    """Stands where HipLib stands when COMPILE_ONLY is set: compiles, never runs."""

    def __init__(self, real: _ffi.HipLib) -> None:
        import sys
        print("dlgrad_amd: DLGRAD_HIP_COMPILE_ONLY=1 -- kernels are compiled, nothing is executed",
              file=sys.stderr)
        self._real, self._next = real, 0x7F0000000000

    def compile(self, *a):
        return self._real.compile(*a)

    def alloc(self, nbytes: int, zero: bool = False) -> int:
        a = self._next
        self._next += (nbytes + 255) // 256 * 256
        return a

    def d2h(self, host_addr: int, src: int, nbytes: int) -> None:
        import ctypes
        ctypes.memset(host_addr, 0, nbytes)

    def module_load(self, code: bytes, name: str) -> int:
        return 1

    def props(self) -> dict:
        return {"name": "compile-only", "arch": K.ARCH, "compute_units": 256, "wavefront_size": 64,
                "clock_khz": 2400000, "mem_clock_khz": 0, "mem_bus_bits": 8192, "lds_bytes": 163840,
                "l2_bytes": 4 << 20, "total_mem": 288 << 30}

    def event_create(self) -> int:
        return 1

    def event_elapsed_ms(self, a: int, b: int) -> float:
        return 1.0

    def pool_stats(self) -> tuple:
        return (0, 0, 0)

    def arena_create(self) -> int:
        return 1

    def graph_end(self) -> tuple:
        return (1, 0)

    def __getattr__(self, name: str):           # free, h2d, launch, sync, fill_f32, events ...
        return lambda *a, **k: None


def _dump_manifest() -> None:
    path = os.environ.get("DLGRAD_HIP_MANIFEST")
    if path and requested_kernels:
        from dlgrad_amd.codegen import manifest
        manifest.merge(requested_kernels, path)


if os.environ.get("DLGRAD_HIP_MANIFEST"):
    import atexit
    atexit.register(_dump_manifest)


try:                                   # the compiled binding of alloc / free / launch (csrc/dlgfast.c)
    from dlgrad_amd import _dlgfast as _fast
except ImportError:                    # not built: the same three calls go through ffi.py's binding
    _fast = None
if os.environ.get("DLGRAD_HIP_FAST_BINDING", "1") == "0":
    _fast = None
_bound = False                         # _fast holds the library's function addresses


def lib() -> _ffi.HipLib:
    """The loaded library with the device initialised; raises when there is no GPU."""
    global _bound
    if not _state["ready"]:
        l = _ffi.get_lib()
        if COMPILE_ONLY:
            l = _CompileOnlyLib(l)
        else:
            l.init(int(os.environ.get("DLGRAD_HIP_DEVICE", "0")))
            if _fast is not None:
                _fast.bind(*[l.function_address(f) for f in ("dlg_hip_alloc", "dlg_hip_free", "dlg_hip_launch",
                                                             "dlg_hip_last_error")])
                _bound = True
        _state["lib"], _state["ready"] = l, True
    return _state["lib"]


def available() -> bool:
    try:
        return _ffi.get_lib().device_count() > 0
    except Exception:
        return False


def props() -> dict:
    if _state["props"] is None:
        _state["props"] = lib().props()
    return _state["props"]


class _PyDevicePtr:
    """An address in HBM.  Owning pointers give their block back to the pool when
    collected; views (`ptr + n_elements`, as tensor.py:816-821 slices) keep their
    base alive instead.  (The form used when the compiled binding is not built.)"""
    __slots__ = ("addr", "nbytes", "base", "__weakref__")

    def __init__(self, addr: int, nbytes: int, base: "DevicePtr | None" = None) -> None:
        self.addr, self.nbytes, self.base = addr, nbytes, base

    def __add__(self, n_elements: int) -> "DevicePtr":
        off = 4 * int(n_elements)
        if off < 0 or off > self.nbytes:
            raise IndexError(f"offset {n_elements} elements outside a {self.nbytes}-byte block")
        return DevicePtr(self.addr + off, self.nbytes - off, self.base or self)

    def __del__(self) -> None:
        if self.base is None and self.addr:
            l = _state["lib"] if _state is not None else None      # module globals are gone at interpreter exit
            if l is not None:
                try:
                    l.free(self.addr)
                except Exception:      # interpreter shutdown
                    pass

    def __repr__(self) -> str:
        return f"DevicePtr(0x{self.addr:x}, {self.nbytes} B{', view' if self.base else ''})"


# The compiled type does the same with its finaliser in C (it calls dlg_hip_free directly); in
# compile-only mode its addresses are made up and nothing is bound, so it frees nothing.
DevicePtr = _fast.DevPtr if _fast is not None else _PyDevicePtr


def alloc(numel: int, zero: bool = False) -> DevicePtr:
    nbytes = 4 * numel if numel > 0 else 4
    if not zero:
        if _bound:
            return _fast.alloc(nbytes)
        l = _state["lib"] or lib()                              # the first call initialises (and binds)
        return _fast.alloc(nbytes) if _bound else DevicePtr(l.alloc(nbytes, False), nbytes)
    if _graph_depth:
        # a memset node must not enter a captured graph: clear with a kernel instead
        p = alloc(numel)
        _map("full", "s0", [], (max(numel, 1),), (0.0,), out=p)
        return p
    return DevicePtr((_state["lib"] or lib()).alloc(nbytes, True), nbytes)


# ---- pinned host staging ------------------------------------------------------------------
_pinned: dict = {}     # address -> bytes of every live page-locked block


def pinned_empty(shape, dtype=np.float32) -> np.ndarray:
    """A numpy array in page-locked host memory.  Uploads from it (Buffer.from_numpy, upload_,
    from_u8) are enqueued without waiting for the copy, and may be recorded into a captured
    graph, which then re-reads the array on every replay.  Do not modify the array between an
    upload and the next sync().  The memory is released when the array is collected."""
    import ctypes
    import weakref
    shape = tuple(shape) if not isinstance(shape, int) else (shape,)
    nbytes = int(np.prod(shape, dtype=np.int64)) * np.dtype(dtype).itemsize
    if COMPILE_ONLY:
        return np.empty(shape, dtype)
    l = lib()
    addr = l.host_alloc(max(nbytes, 1))
    raw = (ctypes.c_char * max(nbytes, 1)).from_address(addr)
    _pinned[addr] = max(nbytes, 1)

    def release(addr=addr):
        _pinned.pop(addr, None)
        cur = _state["lib"]
        if cur is not None:
            try:
                cur.host_free(addr)
            except Exception:      # interpreter shutdown
                pass
    weakref.finalize(raw, release)
    return np.frombuffer(raw, dtype=dtype, count=nbytes // np.dtype(dtype).itemsize).reshape(shape)


def _is_pinned(a: np.ndarray) -> bool:
    p, n = a.ctypes.data, a.nbytes
    return any(b <= p and p + n <= b + size for b, size in _pinned.items())


def _upload(dst_addr: int, a: np.ndarray) -> None:
    """Host array -> device: enqueued without a wait when the array is page-locked."""
    if not a.nbytes:
        return
    if _pinned and _is_pinned(a):
        lib().h2d_async(dst_addr, a.ctypes.data, a.nbytes)
    else:
        lib().h2d(dst_addr, a.ctypes.data, a.nbytes)


# ---- captured graphs ------------------------------------------------------------------------
_graph_depth = 0       # > 0 while a Graph's arena is current (warm-up or capture)
_current_arena = 0     # its id (0: the ordinary pool)
_after_capture: list = []   # host work a captured step deferred until its capture has ended (table uploads)
_capturing = False


def capturing() -> bool:
    return _capturing


def in_graph() -> bool:
    """Whether a Graph's arena is current: the step being issued is a warm-up for a capture, or is being captured."""
    return _graph_depth > 0


class Graph:
    """A whole step -- hundreds of launches -- recorded once and replayed as one submission.

        g = Graph()
        with g.arena():   step()        # eager, inside the graph's private pool: loads every kernel,
                                        # sizes the pool
        with g.capture(): out = step()  # recorded, not executed
        g.replay()                      # runs the recorded launches; `out` is rewritten in place

    What is recorded is the exact launches with their arguments, so the step must keep its
    state at fixed addresses (in-place optimizer), must not transfer to or from the host,
    and anything that changes per replay must live in device memory.  Buffers allocated
    inside arena()/capture() come from a pool nobody else draws from, so replays cannot
    clobber tensors made elsewhere."""

    def __init__(self) -> None:
        self._lib = lib()
        self.arena_id = self._lib.arena_create()
        self.handle, self.nodes = 0, 0

    def _enter(self) -> None:
        global _graph_depth, _current_arena
        if _graph_depth:
            raise RuntimeError("graph arenas do not nest")
        self._lib.arena_set(self.arena_id)
        _graph_depth, _current_arena = 1, self.arena_id

    def _leave(self) -> None:
        global _graph_depth, _current_arena
        _graph_depth, _current_arena = 0, 0
        self._lib.arena_set(0)

    def arena(self):
        import contextlib

        @contextlib.contextmanager
        def cm():
            self._enter()
            try:
                yield self
                self._lib.arena_reserve(self.arena_id)     # blocks for a repeat of this pass, also while its results are held
            finally:
                self._leave()
        return cm()

    def capture(self):
        import contextlib

        @contextlib.contextmanager
        def cm():
            global _capturing
            if self.handle:
                raise RuntimeError("this Graph already holds a capture")
            self._enter()
            self._lib.graph_begin()
            _capturing = True
            try:
                yield self
            except BaseException:
                _capturing = False
                _after_capture.clear()
                self._lib.graph_abandon()
                self._leave()
                raise
            _capturing = False
            try:
                self.handle, self.nodes = self._lib.graph_end()
                for job in _after_capture:
                    job()
            finally:
                _after_capture.clear()
                self._leave()
        return cm()

    def replay(self) -> None:
        global launch_count
        launch_count += 1
        self._lib.graph_launch(self.handle)

    def close(self) -> None:
        if self.handle:
            self._lib.graph_destroy(self.handle)
            self.handle = 0
        if self.arena_id:
            self._lib.arena_destroy(self.arena_id)
            self.arena_id = 0


class CapturedStep:
    """A step function turned into its captured form without the caller handling arenas and captures:

        step = hip.CapturedStep(train_step, before_replay=opt.advance)
        for _ in range(n):
            loss = step()              # 1st call: eager inside the graph's arena; 2nd: recorded and run once; later: one replay each

    Every call performs exactly one step.  The value the function returned while it was recorded is returned by
    every later call: its tensors live at fixed addresses and each replay rewrites them.  before_replay runs ahead of
    every step after the first (the optimizer's advance(), which writes the next step's constants on the device).
    What Graph asks of a step holds here too: state at fixed addresses (in-place optimizer), no host transfers, inputs
    refreshed in place between calls."""

    def __init__(self, fn, before_replay=None) -> None:
        self.fn, self.before_replay = fn, before_replay
        self.graph, self.calls, self.result = Graph(), 0, None

    def __call__(self):
        self.calls += 1
        if self.calls == 1:
            with self.graph.arena():
                return self.fn()
        if self.before_replay is not None:
            self.before_replay()
        if self.calls == 2:
            with self.graph.capture():
                self.result = self.fn()
        self.graph.replay()
        return self.result

    @property
    def nodes(self) -> int:
        return self.graph.nodes

    def close(self) -> None:
        self.graph.close()


# ---- kernel cache -----------------------------------------------------------------------

def code_object(src: str, name: str, l: _ffi.HipLib | None = None, force: bool = False) -> bytes:
    """Code object for `src`: from the on-disk cache, else hiprtc (always hiprtc when `force`,
    which is how the build step recompiles everything).  Needs no GPU."""
    opts = list(K.COMPILE_OPTIONS)
    key = hashlib.sha256((src + "\0" + " ".join(opts)).encode()).hexdigest()[:20]
    path = os.path.join(CACHE_DIR, f"{name}_{key}.hsaco")
    if not force:
        try:
            with open(path, "rb") as f:
                return f.read()
        except FileNotFoundError:
            pass
    code = (l or _ffi.get_lib()).compile(src, name + ".hip", opts)
    compiled_now.append(name)
    os.makedirs(CACHE_DIR, exist_ok=True)
    tmp = f"{path}.{os.getpid()}.tmp"
    with open(tmp, "wb") as f:
        f.write(code)
    os.replace(tmp, path)
    return code


def kernel(gen, *params):
    key = (gen, params)
    h = _handles.get(key)
    if h is None:
        src, name, fmt = gen(*params)
        requested_kernels.add((gen.__name__, params))
        l = lib()
        h = _handles[key] = (l.module_load(code_object(src, name, l), name), struct.Struct(fmt))
        kernel_names[id(h)] = name
    return h


def launch(k, grid, block, *args) -> None:
    """grid / block: an int (x extent) or a 3-tuple."""
    global launch_count
    launch_count += 1
    handle, st = k
    packed = st.pack(*args)
    if grid.__class__ is int:
        gx, gy, gz = grid, 1, 1
    else:
        gx, gy, gz = grid if len(grid) == 3 else (tuple(grid) + (1, 1))[:3]
    if block.__class__ is int:
        bx, by, bz = block, 1, 1
    else:
        bx, by, bz = block if len(block) == 3 else (tuple(block) + (1, 1))[:3]
    if _bound:
        _fast.launch(handle, gx, gy, gz, bx, by, bz, packed)
        return
    l = _state["lib"]
    rc = l.raw_launch(handle, gx, gy, gz, bx, by, bz, 0, packed, len(packed))
    if rc:
        l._check(rc)


def launch_out(k, grid, block, out_offset: int, out_numel: int, *args) -> DevicePtr:
    """A launch whose output is allocated by the same call: `args` holds 0 where the kernel expects
    the output pointer, at byte `out_offset` of its argument block.  grid / block: an int (x extent)
    or a 3-tuple.  Returns the freshly allocated block of out_numel floats."""
    global launch_count
    launch_count += 1
    handle, st = k
    gx, gy, gz = (grid, 1, 1) if grid.__class__ is int else grid
    bx, by, bz = (block, 1, 1) if block.__class__ is int else block
    if _bound:
        return _fast.launch_out(handle, gx, gy, gz, bx, by, bz, st.pack(*args), out_offset, 4 * out_numel if out_numel > 0 else 4)
    out = alloc(out_numel)
    packed = bytearray(st.pack(*args))
    struct.pack_into("@P", packed, out_offset, out.addr)
    l = _state["lib"]
    rc = l.raw_launch(handle, gx, gy, gz, bx, by, bz, 0, bytes(packed), len(packed))
    if rc:
        l._check(rc)
    return out


def field_offset(fmt: str, index: int) -> int:
    """Byte offset of the index-th value of a native-alignment struct format such as "@PPfPI4I"
    (what the kernel generators return; a count repeats its letter)."""
    import re
    assert fmt[0] == "@"
    codes = "".join(c * int(n or 1) for n, c in re.findall(r"(\d*)([a-zA-Z])", fmt[1:]))
    code = codes[index]
    return struct.calcsize("@" + codes[:index] + code) - struct.calcsize("@" + code)


def _addr(b: Buffer) -> int:
    return b.ptr.addr


def _pad4(t: tuple, fill: int) -> tuple:
    return (fill,) * (4 - len(t)) + tuple(t)


# ---- element-wise launcher ------------------------------------------------------------------

class _MapPlan:
    """Everything about one (op, operand shapes) combination that does not depend on the
    addresses: element count, operand modes, the kernel variants and their trailing
    arguments.  Built once, then each call only packs pointers and launches."""
    __slots__ = ("n", "is_scalar", "wide", "narrow")

    def __init__(self, tag: str, expr: str, operands: list, out_shape: tuple, n_svals: int) -> None:
        if len(out_shape) > 4:
            raise ValueError("dlgrad only supports upto 4D tensors")
        n = self.n = prod_(out_shape)
        if n >= 2 ** 31:
            raise ValueError(f"{n} elements exceed the 32-bit index range of the kernels")
        self.is_scalar = tuple(b.is_host_scalar for b in operands)
        self.wide = self.narrow = None
        if n == 0:
            return
        tens = [b for b in operands if not b.is_host_scalar]
        t_strides = [get_broadcast_strides_2(out_shape, b.shape, b.stride) for b in tens]
        cshape, cstr = collapse_dims(out_shape, calculate_stride(out_shape), *t_strides)
        modes: list | None = None
        C = cshape[-1] if len(cshape) == 2 else 1
        if len(cshape) <= 2:
            full = (C, 1) if len(cshape) == 2 else (1,)
            kinds = {full: "vec", (1, 0): "row", (0, 1): "col"}
            it = iter(cstr[1:])
            modes = []
            for sc in self.is_scalar:
                if sc:
                    modes.append("sval")
                    continue
                st = next(it)
                m = "sptr" if not any(st) else kinds.get(st)
                if m is None:
                    modes = None
                    break
                modes.append(m)
        if modes is not None:
            # (generator params, grid, trailing args); the kernel itself is loaded on first use
            if C % 4 == 0 or not any(m in ("row", "col") for m in modes):
                # outputs too large to be re-read from cache are written with nontemporal stores
                # (streaming form: one float4 per thread, which measures 5-8 % above four)
                nt = n >= NT_STORE_MIN_ELEMENTS
                unroll = 1 if nt else 4
                self.wide = [(K.map_kernel, tag, expr, tuple(modes), 4, n_svals, unroll, nt), K.map_grid(n, 4, unroll), (n, C), None,
                             tuple(m in ("vec", "col") for m in modes)]
            self.narrow = [(K.map_kernel, tag, expr, tuple(modes), 1, n_svals), K.map_grid(n, 1), (n, C), None, None]
        else:
            tail = (n, *_pad4(out_shape, 1), *[x for st in t_strides for x in _pad4(st, 0)])
            self.narrow = [(K.strided_map_kernel, tag, expr, len(operands), self.is_scalar, n_svals),
                           (n + 1023) // 1024, tail, None, None]


PLAN_CACHE_ENTRIES = 8192


class _PlanCache(dict):
    """A launch-plan table that cannot grow without bound: a workload whose shapes change on every call (a decoding
    loop whose cache grows by a row per token) would otherwise leave an entry per shape for ever.  Lookups are plain
    dictionary lookups; storing into a full table first drops the older half (insertion order)."""
    __slots__ = ()

    def __setitem__(self, key, value) -> None:
        if len(self) >= PLAN_CACHE_ENTRIES and key not in self:
            for old in list(self)[:PLAN_CACHE_ENTRIES // 2]:
                del self[old]
        dict.__setitem__(self, key, value)


_map_plans: dict = _PlanCache()
EMB_ORDERED = os.environ.get("DLGRAD_HIP_EMB_ORDERED", "1") != "0"     # 0: fp32 atomics for every size
NT_STORE_MIN_ELEMENTS = int(os.environ.get("DLGRAD_HIP_NT_MIN", str(1 << 25)))   # 128 MiB of fp32


def _map(tag: str, expr: str, operands: list[Buffer], out_shape: tuple, svals: tuple = (),
         out: DevicePtr | None = None) -> DevicePtr:
    """Runs `expr` over `operands` broadcast to `out_shape`.

    The iteration space is collapsed jointly over all operands; if what is left is a
    row-major (R, C) grid on which each operand is whole, one-per-row, one-row or a
    single value, the vectorised `map_kernel` runs (16-byte accesses when every pointer
    is 16-byte aligned), otherwise the strided one.  `tag` names `expr` uniquely."""
    key = (tag, out_shape, tuple([None if b.ptr.__class__ is HostScalar else b.metadata.shape for b in operands]),
           len(svals))
    plan = _map_plans.get(key)
    if plan is None:
        plan = _map_plans[key] = _MapPlan(tag, expr, operands, out_shape, len(svals))
    if plan.n == 0:
        return alloc(0) if out is None else out
    args = [float(b.ptr.value) if sc else b.ptr.addr for b, sc in zip(operands, plan.is_scalar)]
    var = plan.wide
    if var is not None:
        if out is not None and out.addr & 15:
            var = plan.narrow
        else:                                  # a fresh output block is at least 256-byte aligned
            for a, needs in zip(args, var[4]):
                if needs and a & 15:
                    var = plan.narrow
                    break
    else:
        var = plan.narrow
    k = var[3]
    if k is None:
        k = var[3] = kernel(*var[0])
        var.append(field_offset(k[1].format, len(operands) + len(svals)))       # where the output pointer goes
    if out is None:                            # output allocation and launch in one call into the library
        return launch_out(k, var[1], 256, var[5], plan.n, *args, *svals, 0, *var[2])
    launch(k, var[1], 256, *args, *svals, out.addr, *var[2])
    return out


_U64 = (1 << 64) - 1
_gemm_plans: dict = _PlanCache()   # the same for products of matrices cut out of larger tensors
_pair_plans: dict = _PlanCache()   # the same for two products that travel as one launch
_matmul_plans: dict = _PlanCache() # (shapes, flags, alignment bits) -> (kernel, grid, threads, fixed arguments, ...) of a product seen before
# short rows of an even length: "direct" = a thread per row with 8-byte loads straight from memory (7.2 us for
# 1 000 000 x 10 against 8.1 for "staged", 256 rows per block through LDS, which remains the form for odd lengths)
ARGMAX_SHORT_ROWS = os.environ.get("DLGRAD_HIP_ARGMAX_SHORT_ROWS", "direct")
ARGMAX_COL_UNROLL = 8              # rows in flight per thread of the column argmax (8192 x 8192: 50.2 us with 4, 49.5 with 8)
# blocks of 64 x 16 threads the first stage of a tall column reduction aims for (16384 x 8192 over axis 0: 88.5 us with 8192,
# 83.6 us = 6.4 TB/s with 2048 -- row chunks of 256 and a quarter of the partials -- 85.8 us with 512)
REDUCE_COL_TX = int(os.environ.get("DLGRAD_HIP_REDUCE_COL_TX", "0"))          # lanes along a row in the blocks of a tall column reduction (0: chosen by size)
REDUCE_COL_BLOCKS = int(os.environ.get("DLGRAD_HIP_REDUCE_COL_BLOCKS", "2048"))
ARGMAX_COL_BLOCKS = 1024           # blocks of 64 x 16 threads the column argmax aims for (8192 x 8192: 65.6 us with 128, 51.5 with 256 or 512, 49.8 with 1024, 57.8 with 2048)
_permute_plans: dict = _PlanCache()
PERMUTE_DIAG = os.environ.get("DLGRAD_HIP_PERMUTE_DIAG", "1") != "0"     # diagonal tile order for power-of-two pitches


class HIP:
    """Dispatch-table entries for Device.HIP."""

    # ---- host boundary ------------------------------------------------------------------------
    @staticmethod
    @dispatcher.register(BufferOps.CREATE, Device.HIP)
    def create(data: np.ndarray, into: Buffer | None = None) -> DevicePtr:
        a = np.ascontiguousarray(data, dtype=np.float32)
        p = into.ptr if into is not None else alloc(a.size)
        _upload(p.addr, a)
        return p

    @staticmethod
    @dispatcher.register(CustomOps.FROM_U8, Device.HIP)
    def from_u8(data: np.ndarray) -> DevicePtr:
        a = np.ascontiguousarray(data, dtype=np.uint8)
        n = a.size
        if n >= 2 ** 32:
            raise ValueError("array too large for 32-bit indexing")
        out = alloc(n)
        if n == 0:
            return out
        raw = alloc((n + 3) // 4)                                # staging for the bytes; freed in stream order
        _upload(raw.addr, a)
        launch(kernel(K.u8_to_f32_kernel), ((n + 3) // 4 + 255) // 256, 256, raw.addr, out.addr, n)
        return out

    @staticmethod
    @dispatcher.register(CustomOps.ROW_STORE, Device.HIP)
    def row_store(dst: Buffer, src: Buffer, idx: Buffer, rows: int, width: int,
                  dst2: Buffer | None = None, src2: Buffer | None = None) -> None:
        """dst2 / src2: a second destination and row of the same shape, stored by the same launch."""
        if not (rows and width):
            return
        if dst2 is None:
            launch(kernel(K.row_store_kernel), (width + 255) // 256, 256, _addr(dst), _addr(src), _addr(idx), rows, width)
        else:
            launch(kernel(K.row_store_kernel, 2), ((width + 255) // 256, 2, 1), 256, _addr(dst), _addr(src), _addr(idx),
                   rows, width, _addr(dst2), _addr(src2))

    # ---- the ends of a decoding step ---------------------------------------------------------------------------------
    @staticmethod
    def decode_qkv_row_fits(x: Buffer, w: Buffer, gain: Buffer, kc: Buffer, vc: Buffer, slot: Buffer) -> bool:
        """One row x against the stacked (3C, K) projection w with the RMSNorm inside, key and value stores of rows of C."""
        C = w.shape[-2] // 3 if w.ndim >= 2 else 0
        return (HIP.DECODE_FUSED and C > 0 and w.shape[-2] == 3 * C and HIP.row_norm_fits(x, w, gain)
                and kc.numel == vc.numel and kc.numel % C == 0 and kc.numel > 0 and slot.numel == 1 and not slot.is_host_scalar)

    @staticmethod
    @dispatcher.register(CustomOps.DECODE_QKV_ROW, Device.HIP)
    def decode_qkv_row(x: Buffer, w: Buffer, gain: Buffer, eps: float, kc: Buffer, vc: Buffer, slot: Buffer) -> DevicePtr:
        """q = (rmsnorm(x) @ w^T)[:C]; the other two thirds of that row go to row (int)slot of kc and vc."""
        if not HIP.decode_qkv_row_fits(x, w, gain, kc, vc, slot):
            raise ValueError(f"decode_qkv_row does not take {x.shape} x {w.shape} into {kc.shape}")
        N, Kd = w.shape[-2:]
        C = N // 3
        out = alloc(C)
        k = kernel(K.row_matmul_nt_kernel, "", K.rmsnorm_plan(Kd, 4), True)
        launch(k, (N + 3) // 4, 256, _addr(x), _addr(w), out.addr, 0, N, Kd, _addr(gain), float(eps),
               _addr(kc), _addr(vc), _addr(slot), C, kc.numel // C)
        return out

    @staticmethod
    @dispatcher.register(CustomOps.DECODE_EMBED, Device.HIP)
    def decode_embed(wte: Buffer, wpe: Buffer, slot: Buffer, T: int, tok: Buffer | None = None, seq: Buffer | None = None,
                     refpos: bool = False):
        """tok given: (x (C floats), hidden (T floats)) for the token tok[0] fed at index slot[0] against T cache rows.
        seq given: x (T * C floats) for the window of the last T tokens of the (rows, 1) token buffer seq."""
        V, C = wte.shape
        P = wpe.shape[0]
        if wpe.shape[1] != C or slot.numel != 1 or slot.is_host_scalar or (tok is None) == (seq is None) or T <= 0:
            raise ValueError(f"decode_embed: tables {wte.shape}, {wpe.shape}, T={T}")
        if seq is not None:
            x = alloc(T * C)
            launch(kernel(K.decode_embed_kernel, True), (T + 3) // 4, 256, _addr(wte), _addr(wpe), _addr(seq), _addr(slot), x.addr,
                   C, V, P, T, seq.numel)
            return x
        x, hidden = alloc(C), alloc(T)
        launch(kernel(K.decode_embed_kernel, False), (T + 64 + 255) // 256, 256, _addr(wte), _addr(wpe), _addr(tok), _addr(slot),
               x.addr, hidden.addr, C, V, P, T, int(bool(refpos)))
        return x, hidden

    @staticmethod
    @dispatcher.register(CustomOps.DECODE_NEXT, Device.HIP)
    def decode_next(logits: Buffer, tok: Buffer, slot: Buffer, seq: Buffer) -> None:
        if not logits.numel or tok.numel != 1 or slot.numel != 1 or tok.is_host_scalar or slot.is_host_scalar:
            raise ValueError(f"decode_next: {logits.shape} logits, token {tok.shape}, index {slot.shape}")
        launch(kernel(K.decode_next_kernel), 1, 256, _addr(logits), _addr(tok), _addr(slot), _addr(seq), logits.numel, seq.numel)

    @staticmethod
    @dispatcher.register(CustomOps.DECODE_SAMPLE, Device.HIP)
    def decode_sample(logits: Buffer, u: Buffer, tok: Buffer, slot: Buffer, seq: Buffer, temperature: float) -> None:
        if not logits.numel or not u.numel or tok.numel != 1 or slot.numel != 1 or tok.is_host_scalar or slot.is_host_scalar \
                or u.is_host_scalar or not float(temperature) > 0.0:
            raise ValueError(f"decode_sample: {logits.shape} logits, {u.shape} uniform numbers, token {tok.shape}, "
                             f"index {slot.shape}, temperature {temperature}")
        launch(kernel(K.decode_sample_kernel), 1, 256, _addr(logits), _addr(u), _addr(tok), _addr(slot), _addr(seq),
               logits.numel, seq.numel, u.numel, float(temperature))

    @staticmethod
    @dispatcher.register(CustomOps.COPY_INTO, Device.HIP)
    def copy_into(dst: Buffer, src: Buffer) -> None:
        if dst.numel:
            lib().d2d(_addr(dst), _addr(src), 4 * dst.numel)

    @staticmethod
    @dispatcher.register(CustomOps.TO_HOST, Device.HIP)
    def to_host(x: Buffer) -> np.ndarray:
        out = np.empty(x.shape, dtype=np.float32)
        if x.numel:
            lib().d2h(out.ctypes.data, _addr(x), 4 * x.numel)
        return out

    @staticmethod
    @dispatcher.register(CustomOps.PRINT, Device.HIP)
    def show(x: Buffer) -> None:
        print(HIP.to_host(x))

    # ---- creation -------------------------------------------------------------------------------
    _seed = int.from_bytes(os.urandom(8), "little")        # the reference reads /dev/random per call
    _stream = 0                                            # one PCG32 stream per uniform() call

    @staticmethod
    def manual_seed(seed: int) -> None:
        """Makes every later uniform() repeatable: call k after this draws PCG32 stream k of `seed`."""
        HIP._seed, HIP._stream = int(seed) & _U64, 0

    @staticmethod
    def _pcg_start(seed: int, seq: int) -> tuple[int, int]:
        """(state, inc) after pcg32_srandom_r(seed, seq) (cpu_kernel.py:829-836)."""
        inc = ((seq << 1) | 1) & _U64
        state = inc                                        # (0 * a + inc)
        state = (state + seed) & _U64
        state = (state * K.PCG32_MULT + inc) & _U64
        return state, inc

    @staticmethod
    def _lcg_jump(delta: int, inc: int) -> tuple[int, int]:
        """(m, p) with state_after_delta_steps = state * m + p  (mod 2^64)."""
        acc_m, acc_p, cur_m, cur_p = 1, 0, K.PCG32_MULT, inc
        while delta:
            if delta & 1:
                acc_m = (acc_m * cur_m) & _U64
                acc_p = (acc_p * cur_m + cur_p) & _U64
            cur_p = ((cur_m + 1) * cur_p) & _U64
            cur_m = (cur_m * cur_m) & _U64
            delta >>= 1
        return acc_m, acc_p

    @staticmethod
    @dispatcher.register(BufferOps.UNIFORM, Device.HIP)
    def uniform(shape: tuple, low: float = 0.0, high: float = 1.0) -> DevicePtr:
        """U[low, high) generated on the device: PCG32 as in cpu_kernel.py:774-874, element i
        being the i-th output of the stream, (float)ldexp(u32, -32), then low + (high-low)*f.
        The reference reseeds from /dev/random on every call; here the seed is the process's
        (random unless manual_seed was called) and each call takes the next stream, so a
        seeded run repeats and successive tensors differ."""
        n = prod_(shape)
        if n >= 2 ** 32:
            raise ValueError("tensor too large for 32-bit indexing")
        if capturing():
            raise RuntimeError("uniform() inside a captured graph would replay the same numbers on every launch")
        out = alloc(n)
        if n == 0:
            return out
        state0, inc = HIP._pcg_start(HIP._seed, HIP._stream)
        HIP._stream += 1
        blocks = min((n + 255) // 256, 4096)
        m, p = HIP._lcg_jump(blocks * 256, inc)
        affine = not (float(low) == 0.0 and float(high) == 1.0)
        launch(kernel(K.uniform_pcg32_kernel), blocks, 256, out.addr, n, state0, inc, m, p, float(low), float(high),
               int(affine))
        return out

    @staticmethod
    @dispatcher.register(BufferOps.FULL, Device.HIP)
    def full(shape: tuple, fill_value: float) -> DevicePtr:
        # cpu.py:252 hands the C kernel int(fill_value)
        v = float(int(fill_value)) if STRICT_REFERENCE else float(fill_value)
        return _map("full", "s0", [], tuple(shape), (v,))

    @staticmethod
    @dispatcher.register(BufferOps.ARANGE, Device.HIP)
    def arange(shape: tuple) -> DevicePtr:
        return _map("arange", "(float)i", [], tuple(shape))

    # ---- binary -----------------------------------------------------------------------------------
    @staticmethod
    def _binary_op(x: Buffer, y: Buffer, op: str) -> DevicePtr:
        return _map(op, K.BINARY_EXPR[op], [x, y], broadcast_shapes_2(x.shape, y.shape))

    @staticmethod
    def _binary_entry(op: str):
        """The dispatch-table entry of one binary op: after the first call for a pair of shapes the launch
        plan is found with one dictionary lookup on (shape, shape) and nothing else is recomputed."""
        expr, plans = K.BINARY_EXPR[op], _PlanCache()

        def run(x: Buffer, y: Buffer) -> DevicePtr:
            xp, yp = x.ptr, y.ptr
            y_host = yp.__class__ is HostScalar
            if xp.__class__ is HostScalar:
                return _map(op, expr, [x, y], broadcast_shapes_2(x.shape, y.shape))
            plan = plans.get((x.shape, None if y_host else y.shape))
            if plan is None:                                   # the general launcher builds and runs it once
                out_shape = broadcast_shapes_2(x.shape, y.shape)
                out = _map(op, expr, [x, y], out_shape)
                plans[(x.shape, None if y_host else y.shape)] = _map_plans[(op, out_shape, (x.shape, None if y_host else y.shape), 0)]
                return out
            if plan.n == 0:
                return alloc(0)
            xa = xp.addr
            ya = float(yp.value) if y_host else yp.addr
            var = plan.wide
            if var is None or (xa & 15 and var[4][0]) or (not y_host and ya & 15 and var[4][1]):
                var = plan.narrow
            k = var[3]
            if k is None:
                return _map(op, expr, [x, y], broadcast_shapes_2(x.shape, y.shape))
            return launch_out(k, var[1], 256, 16, plan.n, xa, ya, 0, *var[2])
        run.__name__ = op
        return run

    add = dispatcher.register(BinaryOps.ADD, Device.HIP)(_binary_entry.__func__("add"))
    sub = dispatcher.register(BinaryOps.SUB, Device.HIP)(_binary_entry.__func__("sub"))
    mul = dispatcher.register(BinaryOps.MUL, Device.HIP)(_binary_entry.__func__("mul"))
    div = dispatcher.register(BinaryOps.DIV, Device.HIP)(_binary_entry.__func__("div"))
    gt = dispatcher.register(BinaryOps.GT, Device.HIP)(_binary_entry.__func__("gt"))
    gte = dispatcher.register(BinaryOps.GTE, Device.HIP)(_binary_entry.__func__("gte"))
    eqt = dispatcher.register(BinaryOps.EQT, Device.HIP)(_binary_entry.__func__("eq"))

    @staticmethod
    @dispatcher.register(BinaryOps.CMP, Device.HIP)
    def cmp(x: Buffer, y: Buffer, out_shape: tuple, mode: str) -> DevicePtr:
        if mode != "<=":
            raise ValueError(f"unsupported comparison {mode!r}")   # cpu.py:839-840 knows only "<="
        return _map("le", K.BINARY_EXPR["le"], [x, y], tuple(out_shape))

    # ---- unary ---------------------------------------------------------------------------------------
    @staticmethod
    def _unary(x: Buffer, tag: str, expr: str, svals: tuple = ()) -> DevicePtr:
        return _map(tag, expr, [x], x.shape, svals)

    @staticmethod
    def _unary_entry(tag: str):
        """The dispatch-table entry of one parameterless unary op: one dictionary lookup on the shape finds the
        launch plan of a call seen before."""
        expr, plans = K.UNARY_EXPR[tag], _PlanCache()

        def run(x: Buffer) -> DevicePtr:
            plan = plans.get(x.shape)
            if plan is None:
                out = _map(tag, expr, [x], x.shape)
                plans[x.shape] = _map_plans[(tag, x.shape, (x.shape,), 0)]
                return out
            xa = x.ptr.addr
            var = plan.narrow if (plan.wide is None or xa & 15) else plan.wide
            k = var[3]
            if k is None or plan.n == 0:
                return _map(tag, expr, [x], x.shape)
            return launch_out(k, var[1], 256, 8, plan.n, xa, 0, *var[2])
        run.__name__ = tag
        return run

    neg = dispatcher.register(UnaryOps.NEG, Device.HIP)(_unary_entry.__func__("neg"))
    exp = dispatcher.register(UnaryOps.EXP, Device.HIP)(_unary_entry.__func__("exp"))
    log = dispatcher.register(UnaryOps.LOG, Device.HIP)(_unary_entry.__func__("log"))
    sqrt = dispatcher.register(UnaryOps.SQRT, Device.HIP)(_unary_entry.__func__("sqrt"))
    rsqrt = dispatcher.register(UnaryOps.RSQRT, Device.HIP)(_unary_entry.__func__("rsqrt"))
    relu = dispatcher.register(UnaryOps.RELU, Device.HIP)(_unary_entry.__func__("relu"))

    @staticmethod
    @dispatcher.register(UnaryOps.POW, Device.HIP)
    def pow(x: Buffer, val: float) -> DevicePtr:
        # cpu.py:500 truncates the exponent to int before the call
        if STRICT_REFERENCE or float(val).is_integer():
            n = int(val)
            return HIP._unary(x, f"pow{n}".replace("-", "m"), K.pow_expr(n))
        return HIP._unary(x, "powf", "powf(x0, s0)", (val,))

    @staticmethod
    @dispatcher.register(UnaryOps.CLAMP, Device.HIP)
    def clamp(x: Buffer, min_val: float | None, max_val: float | None) -> DevicePtr:
        lo, hi = min_val is not None, max_val is not None
        # the reference's two ifs in order (cpu_kernel.py:335-339): v<min -> min, then v>max -> max
        expr, sv = "x0", []
        if lo:
            expr = "((x0 < s0) ? s0 : x0)"
            sv.append(min_val)
        if hi:
            expr = f"(({expr} > s{len(sv)}) ? s{len(sv)} : {expr})"
            sv.append(max_val)
        return HIP._unary(x, f"clamp{int(lo)}{int(hi)}", expr, tuple(sv))

    # ---- selects ----------------------------------------------------------------------------------------
    @staticmethod
    @dispatcher.register(UnaryOps.WHERE, Device.HIP)
    def where(cond: Buffer, x: Buffer, y: Buffer) -> DevicePtr:
        out_shape = broadcast_shapes_2(broadcast_shapes_2(x.shape, y.shape), cond.shape)
        if (cond.ptr.__class__ is DevicePtr and x.ptr.__class__ is DevicePtr and cond.ptr.addr == x.ptr.addr
                and cond.shape == x.shape):
            # relu / leaky_relu call where(t, t, other): read t once
            return _map("where_self", "(x0 > 0.0f) ? x0 : x1", [x, y], out_shape)
        return _map("where", "(x0 > 0.0f) ? x1 : x2", [cond, x, y], out_shape)

    @staticmethod
    @dispatcher.register(UnaryOps.MASKED_FILL, Device.HIP)
    def masked_fill(x: Buffer, mask: Buffer, val: float, out_shape: tuple) -> DevicePtr:
        out_shape = broadcast_shapes_2(x.shape, mask.shape)
        return _map("mfill", "(x1 > 0.0f) ? s0 : x0", [x, mask], out_shape, (val,))

    # ---- reductions ------------------------------------------------------------------------------------
    @staticmethod
    def _reduce_full_into(kop: str, x_addr: int, n: int, divisor: float, out_addr: int) -> None:
        """Two launches: blocks of 2048 vector items (32 KiB) -> partials -> one block; both are
        issued by one call into the library (dlg_hip_reduce_full), the partials in a pool block."""
        global launch_count
        if n == 0:                                       # nothing to add or compare: what the reference's loop leaves in its accumulator
            lib().fill_f32(out_addr, -3.4028234663852886e+38 if kop == "max" else float("nan") if divisor == 0 else 0.0, 1)    # (a mean of nothing is 0 / 0)
            return
        vec = 4 if x_addr % 16 == 0 else 1
        items = (n + vec - 1) // vec
        G = (items + 2047) // 2048
        if G > 65536:                                    # > 537 M elements: fold the partials of the pieces recursively
            part = alloc(G)
            nt = vec == 4 and n >= NT_STORE_MIN_ELEMENTS
            launch(kernel(K.reduce_full_kernel, kop, vec, nt), G, 256, x_addr, part.addr, n, 1.0, 2048)
            HIP._reduce_full_into(kop, part.addr, G, divisor, out_addr)
            return
        nt = G > 1 and vec == 4 and n >= NT_STORE_MIN_ELEMENTS        # streamed once: keep it out of the caches
        k_stage, k_fold = kernel(K.reduce_full_kernel, kop, vec, nt)[0], kernel(K.reduce_full_kernel, kop, 4)[0]
        part = alloc(G) if G > 1 else None
        launch_count += 2 if G > 1 else 1
        (_state["lib"] or lib()).reduce_full(k_stage, k_fold, x_addr, n, vec, float(divisor), out_addr,
                                             part.addr if part is not None else 0, 4 * G if part is not None else 0)

    @staticmethod
    def _reduce_cols(kop: str, x_addr: int, O: int, L: int, I: int, divisor: float, out_addr: int) -> None:
        """Up to 512 rows are folded by one launch of 64x16 blocks.  Taller inputs are split
        into chunks of >= 64 rows (4 loads per thread) so that about REDUCE_COL_BLOCKS blocks exist, which bounds the
        partials at under 1 % of the input; the same kernel then folds the (O, chunks, I) partials."""
        vec = 4 if (I % 4 == 0 and x_addr % 16 == 0 and out_addr % 16 == 0) else 1
        bx = (I + 64 * vec - 1) // (64 * vec)
        ty = 16 if L > 64 else 4
        nt = vec == 4 and O * L * I >= NT_STORE_MIN_ELEMENTS
        # beyond the caches a 32 x 32 block (512 bytes of a row per block) streams better than 64 x 16 (1 KiB): 16384 x 8192 summed
        # over axis 0 at 80 % of the HBM peak against 77 %; wider blocks are worse still (128 x 8: 68 %, 256 x 4: 61 %)
        TX = (REDUCE_COL_TX or (32 if O * L * I >= (1 << 25) else 64)) if (ty == 16 and L > 512) else 64
        if TX != 64:
            ty, bx = 1024 // TX, (I + TX * vec - 1) // (TX * vec)
        k = kernel(K.reduce_cols_kernel, kop, vec, ty, nt, TX)
        chunks = 1 if L <= 512 else max(1, min(REDUCE_COL_BLOCKS // max(1, bx * O), L // 64))
        if chunks == 1:
            launch(k, (bx, 1, O), (TX, ty, 1), x_addr, out_addr, L, I, L, float(divisor))
            return
        chunk = ((L + chunks - 1) // chunks + ty - 1) // ty * ty
        chunks = (L + chunk - 1) // chunk
        part = alloc(O * chunks * I)
        launch(k, (bx, chunks, O), (TX, ty, 1), x_addr, part.addr, L, I, chunk, 1.0)
        HIP._reduce_cols(kop, part.addr, O, chunks, I, divisor, out_addr)

    @staticmethod
    def _reduce(x: Buffer, dim: int, op: str) -> DevicePtr:
        """sum / max / mean over everything (dim -1 or None) or over one axis
        (cpu.py:604-761).  The (outer, L, inner) view of the contiguous input decides
        the kernel: inner == 1 reduces contiguous rows, otherwise columns."""
        kop = "sum" if op == "mean" else op
        if x.numel >= 2 ** 31:
            raise ValueError("tensor too large for 32-bit indexing")
        if dim is None or dim == -1:
            out = alloc(1)
            HIP._reduce_full_into(kop, _addr(x), x.numel, x.numel if op == "mean" else 1.0, out.addr)
            return out
        if dim < 0:
            dim += x.ndim
        O, L, I = prod_(x.shape[:dim]), x.shape[dim], prod_(x.shape[dim + 1:])
        divisor = float(L) if op == "mean" else 1.0
        out = alloc(O * I)
        if O * I == 0:
            return out
        if L == 0:
            # nothing to fold: the reference's loops leave the start value (0, or -FLT_MAX for max), and mean divides it by 0
            start = {"sum": 0.0, "max": -3.4028234663852886e38, "mean": float("nan")}[op]
            return _map("full", "s0", [], (O * I,), (start,), out=out)
        if I == 1:
            if O < 64 and L >= (1 << 16):                  # a few very long rows: full reduction each
                for r in range(O):
                    HIP._reduce_full_into(kop, _addr(x) + 4 * r * L, L, divisor, out.addr + 4 * r)
                return out
            vec = 4 if (L % 4 == 0 and _addr(x) % 16 == 0) else 1
            blk = L >= 2048
            nt = vec == 4 and O * L >= NT_STORE_MIN_ELEMENTS
            launch(kernel(K.reduce_rows_kernel, kop, vec, blk, nt), O if blk else (O + 3) // 4, 256,
                   _addr(x), out.addr, O, L, divisor)
        else:
            if O > 65535:
                raise ValueError("outer extent too large for the column reduction grid")
            HIP._reduce_cols(kop, _addr(x), O, L, I, divisor, out.addr)
        return out

    @staticmethod
    @dispatcher.register(UnaryOps.SUM, Device.HIP)
    def sum(x: Buffer, dim: int) -> DevicePtr:
        return HIP._reduce(x, dim, "sum")

    @staticmethod
    @dispatcher.register(UnaryOps.MEAN, Device.HIP)
    def mean(x: Buffer, dim: int) -> DevicePtr:
        return HIP._reduce(x, dim, "mean")

    @staticmethod
    @dispatcher.register(UnaryOps.MAX, Device.HIP)
    def max(x: Buffer, dim: int, out: Buffer = None) -> DevicePtr:
        return HIP._reduce(x, dim, "max")

    @staticmethod
    @dispatcher.register(UnaryOps.ARGMAX, Device.HIP)
    def argmax(x: Buffer, dim: int) -> DevicePtr:
        if dim is None:
            O, L, I = 1, x.numel, 1                       # cpu.py:913-918 flattens
        else:
            if dim < 0:
                dim += x.ndim
            O, L, I = prod_(x.shape[:dim]), x.shape[dim], prod_(x.shape[dim + 1:])
        out = alloc(O * I)
        if O * I == 0:
            return out
        if L >= 2 ** 31 or O * L * I >= 2 ** 32:
            raise ValueError("tensor too large for 32-bit indexing")
        if I == 1:
            vec = 4 if (L % 4 == 0 and _addr(x) % 16 == 0) else 1
            if L <= 32 and O >= 4096 and ARGMAX_SHORT_ROWS == "direct" and L % 2 == 0 and _addr(x) % 8 == 0:
                cap = 8 if L <= 8 else 16 if L <= 16 else 32
                launch(kernel(K.argmax_kernel, "rows_direct", 1, 4, False, cap), (O + 255) // 256, 256, _addr(x), out.addr, O, L)
            elif L <= 32 and O >= 4096:
                cap = 8 if L <= 8 else 16 if L <= 16 else 32
                wide = 4 if _addr(x) % 16 == 0 else 1
                launch(kernel(K.argmax_kernel, "rows_staged", wide, 4, False, cap), (O + 255) // 256, 256, _addr(x), out.addr, O, L)
            elif L <= 32:
                launch(kernel(K.argmax_kernel, "rows_thread"), (O + 255) // 256, 256, _addr(x), out.addr, O, L)
            elif L < 2048:
                launch(kernel(K.argmax_kernel, "rows_wave", vec), (O + 3) // 4, 256, _addr(x), out.addr, O, L)
            else:
                launch(kernel(K.argmax_kernel, "rows_block", vec, 4, vec == 4 and O * L >= NT_STORE_MIN_ELEMENTS),
                       O, 256, _addr(x), out.addr, O, L)
            return out
        if O > 65535:
            raise ValueError("outer extent too large for the column argmax grid")
        vec = 4 if (I % 4 == 0 and _addr(x) % 16 == 0) else 1
        bx = (I + 64 * vec - 1) // (64 * vec)
        chunks = 1 if L <= 256 else max(1, min(ARGMAX_COL_BLOCKS // max(1, bx * O), L // 64, 65535))
        chunk = (L + chunks - 1) // chunks
        chunks = (L + chunk - 1) // chunk
        k = kernel(K.argmax_kernel, "cols_part", vec, ARGMAX_COL_UNROLL, vec == 4 and O * L * I >= NT_STORE_MIN_ELEMENTS)
        if chunks == 1:
            launch(k, (bx, 1, O), (64, 16, 1), _addr(x), out.addr, 0, 0, L, I, L, 1)
            return out
        pv, pi = alloc(O * chunks * I), alloc(O * chunks * I)
        launch(k, (bx, chunks, O), (64, 16, 1), _addr(x), out.addr, pv.addr, pi.addr, L, I, chunk, 0)
        launch(kernel(K.argmax_kernel, "cols_fin"), ((I + 63) // 64, O), (64, 16, 1), pv.addr, pi.addr, out.addr, O, chunks, I)
        return out

    # ---- permute ---------------------------------------------------------------------------------------------
    @staticmethod
    @dispatcher.register(UnaryOps.TRANSPOSE, Device.HIP)
    def transpose(x: Buffer, dim0: int, dim1: int, out_stride: tuple | None = None, out_shape: tuple | None = None) -> DevicePtr:
        """Materialised swap of two dims, under the name and keywords the reference's other runtimes register
        (cpu_jit.py:316-317, metal.py:374-375; its live CPU runtime routes Buffer.transpose through PERMUTE,
        buffer.py:292-297, as Buffer.transpose does here).  out_stride / out_shape follow from x and are not needed."""
        nd = x.ndim
        d0, d1 = dim0 % nd, dim1 % nd
        order = list(range(nd))
        order[d0], order[d1] = order[d1], order[d0]
        return HIP.permute(x, tuple(order))

    @staticmethod
    @dispatcher.register(UnaryOps.PERMUTE, Device.HIP)
    def permute(x: Buffer, order: tuple) -> DevicePtr:
        """Materialised permutation (cpu.py:333-368).  After merging dims that stay
        adjacent, either the innermost dim is still innermost (strided row copy) or
        another dim became innermost (LDS-tiled transpose of that pair of dims)."""
        n = x.numel
        out = alloc(n)
        if n == 0:
            return out
        key = (x.shape, x.stride, tuple(order))
        plan = _permute_plans.get(key)
        if plan is None:
            plan = _permute_plans[key] = HIP._permute_plan(x.shape, x.stride, order)
        if plan[0] == "gather":
            _, wide_ok, cshape, cin = plan
            vec = 4 if (wide_ok and _addr(x) % 16 == 0 and out.addr % 16 == 0) else 1
            launch(kernel(K.permute_gather_kernel, vec, n >= NT_STORE_MIN_ELEMENTS), (n // vec + 1023) // 1024, 256,
                   _addr(x), out.addr, n // vec, *cshape[:3], cshape[3] // vec, *cin)
            return out
        _, grid, args, grid4, camped, grid128 = plan
        if grid4 and _addr(x) % 16 == 0 and out.addr % 16 == 0:
            if camped and PERMUTE_DIAG:
                big = grid128 >= 1024
                launch(kernel(K.permute_tiled_kernel, 4, 1, 128 if big else 64, n >= NT_STORE_MIN_ELEMENTS),
                       grid128 if big else grid4, 256, _addr(x), out.addr, *args)
            else:
                launch(kernel(K.permute_tiled_kernel, 4), grid4, 256, _addr(x), out.addr, *args)
        else:
            launch(kernel(K.permute_tiled_kernel, 1), grid, 256, _addr(x), out.addr, *args)
        return out

    @staticmethod
    def _permute_plan(shape: tuple, stride: tuple, order: tuple) -> tuple:
        """Everything about a permutation that depends only on shape, strides and order."""
        out_shape = tuple(shape[i] for i in order)
        in_str = tuple(stride[i] for i in order)
        cshape, (cout, cin) = collapse_dims(out_shape, calculate_stride(out_shape), in_str)
        if prod_(shape) == 1 or cin[-1] == 1:
            wide_ok = cshape[-1] % 4 == 0 and all(s % 4 == 0 for s in cin[:-1])
            return "gather", wide_ok, _pad4(cshape, 1), _pad4(cin, 0)
        t = cin.index(1)
        others = [d for d in range(len(cshape) - 1) if d != t]
        ext = [cshape[d] for d in others]
        i_st = [cin[d] for d in others]
        o_st = [cout[d] for d in others]
        while len(ext) < 2:
            ext.insert(0, 1), i_st.insert(0, 0), o_st.insert(0, 0)
        nt, nb = cshape[t], cshape[-1]
        grid = ((nb + 31) // 32) * ((nt + 31) // 32) * ext[0] * ext[1]
        args = (ext[0], ext[1], nt, nb, i_st[0], i_st[1], cin[-1], o_st[0], o_st[1], cout[t])
        # 64 x 64 tiles with 16-byte accesses when every extent and stride is a multiple of 4
        wide = all(v % 4 == 0 for v in (nt, nb, i_st[0], i_st[1], cin[-1], o_st[0], o_st[1], cout[t]))
        grid4 = ((nb + 63) // 64) * ((nt + 63) // 64) * ext[0] * ext[1] if wide else 0
        # an input row pitch that is a multiple of 2 KiB puts the rows of a tile, and the tiles of
        # one block row, on the same few memory channels: those planes are walked diagonally
        camped = bool(wide and (cin[-1] * 4) % 2048 == 0 and (nb + 63) // 64 >= 16)
        grid128 = ((nb + 127) // 128) * ((nt + 127) // 128) * ext[0] * ext[1] if (nt >= 128 and nb >= 128) else 0
        return "tiled", grid, args, grid4, camped, grid128

    # ---- embedding and cross-entropy helpers ----------------------------------------------------------------------
    @staticmethod
    def scatter_small_fits(V: int, W: int, n: int) -> bool:
        """Whether the scatter-add into a (V, W) table from n indices goes out as the one-launch form: a list short
        enough for every row's wavefront to read all of it, and few enough wavefronts."""
        return (EMB_ORDERED and 0 < n <= K.EMB_SMALL_MAX_N and 0 < V and 0 < W
                and V * (((W + 3) // 4 + 63) // 64) <= K.EMB_SMALL_MAX_WAVES and V * W < 2 ** 31)

    @staticmethod
    @dispatcher.register(CustomOps.EMBEDDING, Device.HIP)
    def embedding(x: Buffer, idx: Buffer, out_numel: int, backward: bool = False,
                  upstream_grad: Buffer = None) -> DevicePtr:
        W, n_idx = x.shape[-1], idx.numel
        if backward:
            V = x.numel // W
            if HIP.scatter_small_fits(V, W, n_idx):
                # a small table and a short list: one launch, a wavefront per table row and 64 column items, the reference's order
                out = alloc(x.numel)
                vec = 4 if (W % 4 == 0 and not (_addr(upstream_grad) | out.addr) & 15) else 1
                chunks = (W // vec + 63) // 64
                launch(kernel(K.embedding_backward_small_kernel, vec), (V * chunks + 3) // 4, 256, out.addr, _addr(upstream_grad),
                       _addr(idx), n_idx, W, V, chunks)
                return out
            if n_idx and n_idx <= K.EMB_ORDERED_MAX and EMB_ORDERED and x.numel < 2 ** 31 and W <= 1 << 22:
                # two launches write every element of the table exactly once -- sums in index order where an id
                # occurs, zeros elsewhere -- without a zero-fill pass and without atomics
                NS = (n_idx + K.EMB_SEGMENT - 1) // K.EMB_SEGMENT
                out, partial, segmask, firsts, idsegs = alloc(x.numel), alloc(n_idx * W), alloc(2 * n_idx), alloc(n_idx * NS), alloc(2 * V)
                gfirst = alloc(n_idx)
                vec = 4 if (W % 4 == 0 and not (_addr(upstream_grad) | out.addr | partial.addr) & 15) else 1
                n_sum, n_zero = (n_idx + 3) // 4, (V + 63) // 64
                every = max(1, (n_sum + n_zero) // n_zero)     # one zero block among every so many
                launch(kernel(K.embedding_backward_ordered_kernel, "mark", 1, False, 4 if _addr(idx) % 16 == 0 else 1),
                       n_zero, 256, idsegs.addr, _addr(idx), n_idx, V)
                launch(kernel(K.embedding_backward_ordered_kernel, "segments", vec, x.numel >= NT_STORE_MIN_ELEMENTS),
                       n_sum + n_zero, 256, out.addr, partial.addr, segmask.addr, firsts.addr, gfirst.addr, idsegs.addr,
                       _addr(upstream_grad), _addr(idx), n_idx, W, V, n_zero, every)
                if NS > 1:                                     # (within one segment no id spans segments: nothing to merge)
                    launch(kernel(K.embedding_backward_ordered_kernel, "merge", vec), n_sum, 256, out.addr, partial.addr,
                           segmask.addr, firsts.addr, gfirst.addr, _addr(idx), n_idx, W, V)
                return out
            out = alloc(x.numel, zero=True)                    # init_with_scalar(0), cpu.py:1031
            if n_idx:                                          # very long index lists: hardware fp32 atomics
                launch(kernel(K.embedding_backward_kernel), (n_idx + 3) // 4, 256,
                       out.addr, _addr(upstream_grad), _addr(idx), n_idx, W, V)
            return out
        out = alloc(out_numel)
        if n_idx:
            aligned = int(W % 4 == 0 and _addr(x) % 16 == 0 and out.addr % 16 == 0)
            launch(kernel(K.embedding_kernel), (n_idx + 3) // 4, 256,
                   _addr(x), _addr(idx), out.addr, n_idx, W, aligned, x.numel)
        return out

    @staticmethod
    @dispatcher.register(CustomOps.EMBEDDING_SUM, Device.HIP)
    def embedding_sum(tok_table: Buffer, pos_table: Buffer, idx: Buffer, pos: Buffer) -> DevicePtr:
        """out[i] = tok_table[idx[i]] + pos_table[pos[i % T]] for the idx.numel positions (T = pos.numel)."""
        W, n, T = tok_table.shape[-1], idx.numel, pos.numel
        if pos_table.shape[-1] != W or T == 0 or n % T or max(tok_table.numel, pos_table.numel, n * W) >= 2 ** 31:
            raise ValueError(f"embedding_sum: tables {tok_table.shape}, {pos_table.shape}, {n} ids, {T} positions")
        out = alloc(n * W)
        if n:
            aligned = int(W % 4 == 0 and not (_addr(tok_table) | _addr(pos_table) | out.addr) & 15)
            launch(kernel(K.embedding_sum_kernel), (n + 3) // 4, 256, _addr(tok_table), _addr(pos_table), _addr(idx), _addr(pos),
                   out.addr, n, T, W, tok_table.numel, pos_table.numel, aligned)
        return out

    @staticmethod
    @dispatcher.register(CustomOps.CE_FORWARD, Device.HIP)
    def ce_forward(x: Buffer, y: Buffer) -> DevicePtr:
        rows = x.shape[0]
        out = alloc(rows)
        launch(kernel(K.ce_kernel, False), (rows + 255) // 256, 256, _addr(x), _addr(y), out.addr,
               rows, x.stride[0], x.shape[-1])
        return out

    @staticmethod
    @dispatcher.register(CustomOps.CE_BACKWARD, Device.HIP)
    def ce_backward(x: Buffer, target: Buffer) -> None:
        rows = x.shape[0]
        launch(kernel(K.ce_kernel, True), (rows + 255) // 256, 256, _addr(x), _addr(target), rows, x.stride[0], x.shape[-1])

    # ---- fused row softmax / cross-entropy ------------------------------------------------------------------------------
    @staticmethod
    def _softmax(x: Buffer, dim: int, log: bool, target: Buffer | None = None):
        if dim < 0:
            dim += x.ndim
        if dim != x.ndim - 1:
            raise ValueError("the fused softmax kernel reduces the last axis only")
        L = x.shape[-1]
        R = x.numel // max(L, 1)
        out = alloc(x.numel)
        picked = alloc(R) if target is not None else None
        if x.numel == 0:
            return out if target is None else (out, picked)
        vec = 4 if (L % 4 == 0 and _addr(x) % 16 == 0 and out.addr % 16 == 0) else 1
        blk, nval, threads = K.softmax_plan(L, vec)
        k = kernel(K.softmax_rows_kernel, log, vec, blk, nval, target is not None, threads,
                   x.numel >= NT_STORE_MIN_ELEMENTS)
        grid = R if blk else (R + 3) // 4
        if target is None:
            launch(k, grid, threads, _addr(x), out.addr, R, L)
            return out
        launch(k, grid, threads, _addr(x), out.addr, R, L, _addr(target), picked.addr)
        return out, picked

    @staticmethod
    @dispatcher.register(CustomOps.SOFTMAX, Device.HIP)
    def softmax(x: Buffer, dim: int) -> DevicePtr:
        return HIP._softmax(x, dim, False)

    @staticmethod
    def softmax_bwd_fits(y: Buffer, g: Buffer) -> bool:
        L = y.shape[-1] if y.ndim else 0
        if not L or g.numel != y.numel or g.is_host_scalar:
            return False
        return K.rmsnorm_plan(L, HIP._rms_vec(L, _addr(y), _addr(g))) > 0

    @staticmethod
    @dispatcher.register(CustomOps.SOFTMAX_BWD, Device.HIP)
    def softmax_bwd(y: Buffer, g: Buffer) -> DevicePtr:
        L = y.shape[-1]
        R = y.numel // L
        dx = alloc(y.numel)
        vec = HIP._rms_vec(L, _addr(y), _addr(g), dx.addr)
        nval = K.rmsnorm_plan(L, vec)
        if nval == 0 or g.numel != y.numel:
            raise ValueError(f"fused softmax backward does not take rows of {L} floats here")
        launch(kernel(K.softmax_bwd_rows_kernel, vec, nval, y.numel >= NT_STORE_MIN_ELEMENTS), (R + 3) // 4, 256,
               _addr(y), _addr(g), dx.addr, R, L)
        return dx

    @staticmethod
    def _mask_rows(x: Buffer, mask: Buffer) -> int:
        """How many rows of x.shape[-1] floats the mask has if it lines up with the trailing dims
        of a contiguous x (row r of x then uses mask row r % rows), else 0."""
        if x.ndim == 0 or mask.is_host_scalar or not mask.numel:
            return 0
        L = x.shape[-1]
        mshape = tuple(mask.shape)
        while len(mshape) > 1 and mshape[0] == 1:
            mshape = mshape[1:]
        if len(mshape) > x.ndim or mshape != tuple(x.shape[x.ndim - len(mshape):]):
            return 0
        if tuple(mask.stride) != tuple(calculate_stride(mask.shape)):
            return 0
        return mask.numel // L

    @staticmethod
    def masked_softmax_fits(x: Buffer, mask: Buffer) -> bool:
        """The fused scaled, masked softmax takes rows that the register-resident softmax and its
        one-wavefront backward hold, and a contiguous mask shaped like the trailing dims of x."""
        if not x.numel or not HIP._mask_rows(x, mask):
            return False
        L = x.shape[-1]
        vec = HIP._rms_vec(L, _addr(x), _addr(mask))
        return K.softmax_plan(L, vec)[1] > 0 and K.rmsnorm_plan(L, vec) > 0

    @staticmethod
    def causal_softmax_fits(T: int) -> bool:
        """Whether rows of T scores fit the fused masked softmax and its backward (fresh
        allocations are 256-byte aligned, so only T decides the access width)."""
        vec = 4 if T % 4 == 0 else 1
        return T > 0 and K.softmax_plan(T, vec)[1] > 0 and K.rmsnorm_plan(T, vec) > 0

    @staticmethod
    @dispatcher.register(CustomOps.MASKED_SOFTMAX, Device.HIP)
    def masked_softmax(x: Buffer, mask: Buffer, scale: float) -> DevicePtr:
        """softmax over the last axis of x * scale with -inf where mask > 0: the three kernels of
        `(att * scale).masked_fill(mask, -inf).softmax(dim)` (examples/gpt.py:51-54) as one,
        same arithmetic in the same order."""
        L = x.shape[-1]
        R = x.numel // L
        mrows = HIP._mask_rows(x, mask)
        out = alloc(x.numel)
        vec = HIP._rms_vec(L, _addr(x), _addr(mask), out.addr)
        blk, nval, threads = K.softmax_plan(L, vec)
        if not mrows or not nval:
            raise ValueError(f"fused masked softmax does not take x {x.shape} with mask {mask.shape}")
        how = "causal" if vec == 4 and HIP._is_causal_mask(mask, L, mrows) else True
        k = kernel(K.softmax_rows_kernel, False, vec, blk, nval, False, threads, x.numel >= NT_STORE_MIN_ELEMENTS, how)
        launch(k, R if blk else (R + 3) // 4, threads, _addr(x), out.addr, R, L, _addr(mask), mrows, float(scale))
        return out

    @staticmethod
    def _is_causal_mask(mask: Buffer, L: int, mrows: int) -> bool:
        """Whether `mask` is the (L, L) causal mask this package built and keeps (ops.causal_mask): its contents are then
        known -- 1 where column > row -- and the softmax kernels compute them instead of reading them."""
        if not HIP.CAUSAL_MASK_KNOWN or mrows != L:
            return False
        from dlgrad_amd.ops import _causal_masks
        kept = _causal_masks.get((L, Device.HIP))
        return kept is not None and kept.ptr is mask.ptr

    @staticmethod
    @dispatcher.register(CustomOps.MASKED_SOFTMAX_BWD, Device.HIP)
    def masked_softmax_bwd(y: Buffer, g: Buffer, mask: Buffer, scale: float) -> DevicePtr:
        """(mask > 0 ? 0 : y * (g - sum(g * y))) * scale: the backward nodes of softmax,
        masked_fill and the multiplication by a scalar in one kernel."""
        L = y.shape[-1]
        R = y.numel // L
        mrows = HIP._mask_rows(y, mask)
        dx = alloc(y.numel)
        vec = HIP._rms_vec(L, _addr(y), _addr(g), _addr(mask), dx.addr)
        nval = K.rmsnorm_plan(L, vec)
        if not mrows or nval == 0 or g.numel != y.numel or g.is_host_scalar:
            raise ValueError(f"fused masked softmax backward does not take y {y.shape} with mask {mask.shape}")
        how = "causal" if vec == 4 and HIP._is_causal_mask(mask, L, mrows) else True
        launch(kernel(K.softmax_bwd_rows_kernel, vec, nval, y.numel >= NT_STORE_MIN_ELEMENTS, how), (R + 3) // 4, 256,
               _addr(y), _addr(g), dx.addr, R, L, _addr(mask), mrows, float(scale))
        return dx

    @staticmethod
    @dispatcher.register(CustomOps.LOG_SOFTMAX, Device.HIP)
    def log_softmax(x: Buffer, dim: int) -> DevicePtr:
        return HIP._softmax(x, dim, True)

    @staticmethod
    @dispatcher.register(CustomOps.LOG_SOFTMAX_GATHER, Device.HIP)
    def log_softmax_gather(x: Buffer, target: Buffer) -> tuple[DevicePtr, DevicePtr]:
        """log-softmax over the rows of a 2-D x and, in the same kernel, the ce_forward
        gather picked[i] = lsm[i, (int)target[i]] (cpu.py:961-981)."""
        return HIP._softmax(x, x.ndim - 1, True, target)

    @staticmethod
    @dispatcher.register(CustomOps.CE_GRAD, Device.HIP)
    def ce_grad(lsm: Buffer, target: Buffer, upstream: Buffer, n: float) -> DevicePtr:
        """((exp(lsm) - onehot(target)) * upstream) / n in one pass: the four kernels of
        CrossEntropy.backward (exp, in-place ce_backward, mul, div; ops.py:359-370) fused.
        Same operation order, so it differs from them only through expf."""
        rows = Buffer(target.ptr, (lsm.shape[0], 1), Device.HIP)
        # the column of element i is i % C only while the launcher keeps the (rows, V) grid: a single
        # row collapses to a flat run whose C is 1, and there the column is i itself
        one = lsm.shape[0] == 1
        col = "i" if one else "(i % C)"
        expr = "((expf(x0) - ((" + col + " == (u32)(int)x1) ? 1.0f : 0.0f)) * {g}) / s0"
        tag = "cegrad1" if one else "cegrad"
        if upstream.is_host_scalar:
            return _map(tag + "_v", expr.format(g="s1"), [lsm, rows], lsm.shape,
                        (n, float(upstream.ptr.value)))
        return _map(tag + "_p", expr.format(g="x2"), [lsm, rows, upstream], lsm.shape, (n,))

    @staticmethod
    def ce_stats_fits(x: Buffer) -> bool:
        return x.ndim == 2 and 0 < x.numel < 2 ** 31

    @staticmethod
    @dispatcher.register(CustomOps.CE_STATS, Device.HIP)
    def ce_stats(x: Buffer, target: Buffer, negate: bool = False) -> tuple[DevicePtr, DevicePtr, DevicePtr]:
        """(max, log(sum(exp(x - max))), (x[target] - max) - logsum) per row of the 2-D logits x: all
        the forward pass of the cross-entropy loss needs (ops.py:337-357), from one read of x and with
        no (N, V) intermediate.  negate: the third array holds the row losses -((x[target] - max) - logsum)."""
        R, L = x.shape
        m, ls, picked = alloc(R), alloc(R), alloc(R)
        vec = 4 if (L % 4 == 0 and _addr(x) % 16 == 0) else 1
        blk = L >= 2048
        k = kernel(K.ce_stats_kernel, vec, blk, x.numel >= NT_STORE_MIN_ELEMENTS, bool(negate))
        launch(k, R if blk else (R + 3) // 4, 256, _addr(x), _addr(target), m.addr, ls.addr, picked.addr, R, L)
        return m, ls, picked

    @staticmethod
    @dispatcher.register(CustomOps.CE_GRAD_LOGITS, Device.HIP)
    def ce_grad_logits(x: Buffer, m: Buffer, ls: Buffer, target: Buffer, upstream: Buffer, n: float) -> DevicePtr:
        """((exp((x - m) - ls) - onehot(target)) * upstream) / n in one pass over the logits: the
        log-softmax entry is rebuilt from the row statistics ce_stats kept (the same two subtractions
        on the same values the stored tensor was made with), then the four kernels of
        CrossEntropy.backward (exp, in-place ce_backward, mul, div; ops.py:359-370) follow fused."""
        R, C = x.shape
        # a power of two divides exactly as its reciprocal multiplies (1 / n stays a normal number up to 2^126)
        pow2 = 1.0 <= n <= 2.0 ** 126 and math.frexp(n)[0] == 0.5
        items = 1 if C <= 1024 else 2 if (C <= 2048 or pow2) else 4     # (without the division two loads per thread go faster than four)
        runs = -(-C // (1024 * items))
        if HIP.CE_GRAD_ROWS and C % 4 == 0 and not (_addr(x) & 15) and 0 < R * runs < 2 ** 31 and x.numel < 2 ** 31:
            # a block per (row, run of columns): the row's statistics are read once per block and no index is divided
            by_value = upstream.is_host_scalar
            k = kernel(K.ce_grad_rows_kernel, items, x.numel >= NT_STORE_MIN_ELEMENTS, by_value, pow2)
            g = float(upstream.ptr.value) if by_value else _addr(upstream)
            return launch_out(k, R * runs, 256, field_offset(k[1].format, 5), x.numel, _addr(x), _addr(m), _addr(ls), _addr(target),
                              g, 0, C, runs, 1.0 / n if pow2 else float(n))
        rows = [Buffer(b.ptr, (R, 1), Device.HIP) for b in (m, ls, target)]
        one = R == 1                                     # a single row collapses to a flat run: the column is i itself
        col = "i" if one else "(i % C)"
        expr = "((expf((x0 - x1) - x2) - ((" + col + " == (u32)(int)x3) ? 1.0f : 0.0f)) * {g}) / s0"
        tag = "cegradx1" if one else "cegradx"
        if upstream.is_host_scalar:
            return _map(tag + "_v", expr.format(g="s1"), [x, *rows], x.shape, (n, float(upstream.ptr.value)))
        return _map(tag + "_p", expr.format(g="x4"), [x, *rows, upstream], x.shape, (n,))

    # ---- fused RMSNorm ------------------------------------------------------------------------------------------------------
    @staticmethod
    def rmsnorm_fits(x: Buffer, w: Buffer | None) -> bool:
        """Whether the fused kernels apply: rows of the last axis fit a wavefront's registers
        and the weight, if any, is one row of that length."""
        L = x.shape[-1] if x.ndim else 0
        if x.ndim < 1 or L == 0 or x.numel >= 2 ** 31 or (w is not None and w.numel != L):
            return False
        return K.rmsnorm_plan(L, HIP._rms_vec(L, _addr(x), _addr(w) if w is not None else 0)) > 0

    @staticmethod
    def _rms_vec(L: int, *addrs: int) -> int:
        return 4 if (L % 4 == 0 and all(a % 16 == 0 for a in addrs)) else 1

    @staticmethod
    @dispatcher.register(CustomOps.RMSNORM, Device.HIP)
    def rmsnorm(x: Buffer, w: Buffer | None, eps: float) -> tuple[DevicePtr, DevicePtr]:
        L = x.shape[-1]
        R = x.numel // L
        y, r = alloc(x.numel), alloc(R)
        if not HIP.rmsnorm_fits(x, w):
            raise ValueError(f"fused RMSNorm does not take rows of {L} floats with this weight")
        vec = HIP._rms_vec(L, _addr(x), y.addr, _addr(w) if w is not None else 0)
        nval = K.rmsnorm_plan(L, vec)
        if nval == 0:
            raise ValueError(f"fused RMSNorm: a row of {L} unaligned floats does not fit a wavefront's registers")
        k = kernel(K.rmsnorm_fwd_kernel, vec, nval, w is not None)
        launch(k, (R + 3) // 4, 256, _addr(x), _addr(w) if w is not None else 0, y.addr, r.addr, R, L, float(eps))
        return y, r

    @staticmethod
    @dispatcher.register(CustomOps.RMSNORM_BWD, Device.HIP)
    def rmsnorm_bwd(x: Buffer, w: Buffer | None, r: Buffer, dy: Buffer,
                    through_mean: bool, plus: Buffer | None = None, partial_dw: bool = False) -> tuple:
        """plus: an array shaped like x that is added to dx as it is stored (a gradient that reached x by another route).
        partial_dw: where one column-sum launch would finish dw, hand back (partial rows, their count) instead of
        running it, so that the caller can leave the sum pending."""
        L = x.shape[-1]
        R = x.numel // L
        if dy.numel != x.numel or r.numel != R:
            raise ValueError(f"rmsnorm_bwd: x {x.shape}, dy {dy.shape}, r {r.shape} do not agree")
        if _addr(dy) % 16 and L % 4 == 0:                          # a gradient view at an odd offset: realign it
            dy = Buffer(_map("copy", "x0", [dy], dy.shape), dy.shape, Device.HIP)
        dx = alloc(x.numel)
        # partial rows of dw: at most 2048, and for small inputs (launch-bound) at most the 512 that one launch folds
        rows_per_wave = max(1, (R + 511) // 512 if R * L <= (1 << 20) else (R + 2047) // 2048)
        P = (R + rows_per_wave - 1) // rows_per_wave            # partial rows of dw, one per wavefront
        part = alloc(P * L) if w is not None else None
        if plus is not None and (plus.numel != x.numel or plus.is_host_scalar):
            raise ValueError(f"rmsnorm_bwd: plus {plus.shape} is not shaped like x {x.shape}")
        vec = HIP._rms_vec(L, _addr(x), _addr(dy), dx.addr, _addr(w) if w is not None else 0,
                           part.addr if part is not None else 0, _addr(plus) if plus is not None else 0)
        nval = K.rmsnorm_plan(L, vec)
        if nval == 0:
            raise ValueError(f"fused RMSNorm: a row of {L} unaligned floats does not fit a wavefront's registers")
        k = kernel(K.rmsnorm_bwd_kernel, vec, nval, w is not None, bool(through_mean), plus is not None)
        launch(k, (P + 3) // 4, 256, _addr(x), _addr(w) if w is not None else 0, _addr(r), _addr(dy), dx.addr,
               part.addr if part is not None else 0, R, L, rows_per_wave, *([_addr(plus)] if plus is not None else []))
        if w is None:
            return dx, None
        if partial_dw and 1 < P <= 512:
            return dx, (part, P)
        dw = alloc(L)
        HIP._reduce_cols("sum", part.addr, 1, P, L, 1.0, dw.addr)
        return dx, dw

    # ---- fused optimizer step -----------------------------------------------------------------------------------------------
    @staticmethod
    @dispatcher.register(CustomOps.ADAM_STEP, Device.HIP)
    def adam_step(p: Buffer, g: Buffer, m: Buffer, v: Buffer, consts: tuple) -> tuple[DevicePtr, DevicePtr, DevicePtr]:
        """consts = (b1, 1-b1, b2, 1-b2, 1-b1^t, 1-b2^t, eps, lr), each rounded to fp32 exactly
        where the op-by-op path rounds it (a Python float entering a kernel by value)."""
        n = p.numel
        outs = (alloc(n), alloc(n), alloc(n))
        if n == 0:
            return outs
        addrs = [_addr(b) for b in (p, g, m, v)] + [o.addr for o in outs]
        vec = 4 if not any(a & 15 for a in addrs) else 1
        launch(kernel(K.adam_kernel, vec), max(1, ((n + vec - 1) // vec + 255) // 256), 256,
               *addrs, n, *[float(c) for c in consts])
        return outs

    @staticmethod
    @dispatcher.register(CustomOps.ADAM_STEP_INPLACE, Device.HIP)
    def adam_step_inplace(p: Buffer, g: Buffer, m: Buffer, v: Buffer, consts: Buffer) -> None:
        """Updates p, m and v where they are; `consts` is a device buffer of the eight values
        adam_step takes by value."""
        n = p.numel
        if n == 0:
            return
        addrs = [_addr(b) for b in (p, g, m, v)]
        vec = 4 if not any(a & 15 for a in addrs) else 1
        launch(kernel(K.adam_inplace_kernel, vec), max(1, ((n + vec - 1) // vec + 255) // 256), 256,
               *addrs, n, _addr(consts))

    _stage: dict = {"slots": [], "events": [], "next": 0}

    @staticmethod
    def _stage_upload(bufs: list, arrays: list) -> None:
        """Uploads small host arrays into device buffers without waiting: they are copied into one of four page-locked
        staging blocks and the copies are enqueued on the stream, in order with the launches around them.  A staging
        block is reused only after the copies issued from it have finished (an event per block, normally long done)."""
        st, l = HIP._stage, lib()
        if st.get("lib") is not l:                           # a library that was shut down took its blocks and events with it
            st.update(slots=[], events=[], next=0, lib=l)
        need = sum(a.size for a in arrays)
        i = st["next"]
        st["next"] = (i + 1) % 4
        if len(st["slots"]) <= i:
            st["slots"].append(pinned_empty((max(need, 4096),)))
            st["events"].append(l.event_create())
        else:
            l.event_sync(st["events"][i])
            if st["slots"][i].size < need:
                st["slots"][i] = pinned_empty((2 * need,))
        slot, at = st["slots"][i], 0
        for b, a in zip(bufs, arrays):
            if a.size:
                slot[at:at + a.size] = a.reshape(-1)
                l.h2d_async(b.addr, slot[at:at + a.size].ctypes.data, a.nbytes)
                at += a.size
        l.event_record(st["events"][i])

    @staticmethod
    @dispatcher.register(CustomOps.ADAM_MULTI_INPLACE, Device.HIP)
    def adam_multi_inplace(tensors: list, consts: Buffer, table: dict | None) -> dict:
        """tensors: (p, g, m, v) Buffers per parameter.  `table` is what the previous call
        returned: the device-side address table is rewritten (a host-to-device upload) only when
        some address differs from it.  A table written for a captured step is never touched
        again (the caller keeps it alive as long as the graph); later eager steps get their own.
        A gradient that is a pending sum (buffer.PartialSum) is taken as its parts: the kernel adds
        them up as it reads, in the order of the column-sum launch that would otherwise have run."""
        from dlgrad_amd.buffer import PartialSum
        rows_of = []                                     # per tensor: how many parts the gradient pointer holds, and how far apart
        addrs = []
        low = 0                                          # the low address bits of all tensors, or-ed
        for pb, gb, mb, vb in tensors:
            if gb.__class__ is PartialSum and gb.pending:
                g_addr, rows, pitch = gb.parts.ptr.addr + 4 * gb.offset, gb.parts.shape[0], gb.pitch
                if pitch >= 2 ** 32 or pitch & 3 and not pb.numel & 3:
                    raise ValueError("adam_multi_inplace: parts of a pending gradient lie too far apart or break the 16-byte alignment")
                rows_of += (rows, pitch)
            else:
                g_addr = gb.ptr.addr
                rows_of += (1, 0)
            quad = (pb.ptr.addr, g_addr, mb.ptr.addr, vb.ptr.addr)
            low |= quad[0] | g_addr | quad[2] | quad[3]
            addrs += quad
        addrs = tuple(addrs)
        if low & 15:
            raise ValueError("adam_multi_inplace needs 16-byte aligned tensors")
        key = (addrs, tuple(rows_of))
        if table is None or table["key"] != key:
            nt = len(tensors)
            layout = (key[1], tuple(q[0].numel for q in tensors))
            ptrs = np.array(addrs, dtype=np.uint64).reshape(nt, 4).T.reshape(-1).view(np.float32)        # four rows: p, g, m, v (raw bits)
            if (table is not None and not table["frozen"] and table["layout"] == layout
                    and not capturing() and not _graph_depth and not COMPILE_ONLY):
                # an eager step whose tensors only moved: the sizes and the split into blocks stand, the addresses are sent again
                HIP._stage_upload(table["bufs"][:1], [ptrs])
                table["key"] = key
            else:
                sizes = np.array(layout[1], dtype=np.uint32)
                # 256 threads take 256 16-byte items -- or 16 of them, sharing the addition of a gradient that is pending in many parts
                per_block = np.array([16 if (r > 16 and not n & 3) else 256 for r, n in zip(rows_of[::2], sizes)], dtype=np.int64)
                nblk = np.maximum(1, (sizes.astype(np.int64) // 4 + per_block - 1) // per_block)
                first = np.concatenate([[0], np.cumsum(nblk)[:-1]]).astype(np.uint32)
                owner = np.repeat(np.arange(nt, dtype=np.uint32), nblk)
                arrays = [ptrs] + [np.ascontiguousarray(a).view(np.float32)
                                   for a in (sizes, first, owner, np.array(rows_of, dtype=np.uint32))]     # raw bits; rows_of holds (parts, pitch) pairs
                reuse = (table is not None and not table["frozen"]
                         and [a.size for a in arrays] == [b.nbytes // 4 for b in table["bufs"]])
                bufs = table["bufs"] if reuse else [alloc(a.size) for a in arrays]

                def upload(bufs=bufs, arrays=arrays):
                    for b, a in zip(bufs, arrays):
                        if a.size:
                            lib().h2d(b.addr, a.ctypes.data, a.nbytes)
                if capturing():
                    # a captured launch only records where the table is; its contents are written once the
                    # capture has ended, and never again: the graph replays with exactly these addresses
                    _after_capture.append(upload)
                elif _graph_depth or COMPILE_ONLY:
                    upload()
                else:
                    HIP._stage_upload(bufs, arrays)                # an eager step: enqueued, the host does not wait
                table = {"key": key, "layout": layout, "grid": int(nblk.sum()), "nt": nt, "bufs": bufs, "frozen": capturing()}
        if table["nt"]:
            b = table["bufs"]
            launch(kernel(K.adam_multi_inplace_kernel), table["grid"], 256, b[0].addr, b[1].addr, b[2].addr, b[3].addr, b[4].addr,
                   table["nt"], _addr(consts))
        return table

    @staticmethod
    @dispatcher.register(CustomOps.SET_VALUES, Device.HIP)
    def set_values(dst: Buffer, values: tuple) -> None:
        """dst[i] = values[i] for up to eight Python floats, written by a launch: unlike an upload the host
        does not wait for the stream, and the values are ordered with the kernels around them.  Inside a
        capture the values would be frozen into the graph, so it is refused there."""
        n = len(values)
        if not 0 < n <= 8 or dst.numel < n:
            raise ValueError(f"set_values: {n} values into a buffer of {dst.numel}")
        if capturing():
            raise RuntimeError("set_values inside a captured graph would replay the same values on every launch")
        expr = " : ".join(f"(i == {k}u) ? s{k}" for k in range(n - 1)) + (" : " if n > 1 else "") + f"s{n - 1}"
        _map(f"set{n}", expr, [], (n,), tuple(float(v) for v in values), out=dst.ptr)

    @staticmethod
    @dispatcher.register(CustomOps.SGD_STEP_INPLACE, Device.HIP)
    def sgd_step_inplace(p: Buffer, g: Buffer, v: Buffer | None, lr: float, momentum: float) -> None:
        n = p.numel
        if n == 0:
            return
        if g.numel != n or (v is not None and v.numel != n):
            raise ValueError(f"sgd_step_: parameter {p.shape}, gradient {g.shape}")
        launch(kernel(K.sgd_inplace_kernel, v is not None), (n + 255) // 256, 256,
               _addr(p), _addr(g), _addr(v) if v is not None else 0, n, float(lr), float(momentum))

    @staticmethod
    def sgd_multi_inplace(triples: list, lr: float, momentum: float) -> None:
        """The in-place SGD update of every (p, g, v) triple (v None without momentum) in launches of up to
        K.SGD_MULTI_MAX parameters each; addresses and sizes travel as kernel arguments."""
        M = K.SGD_MULTI_MAX
        live = []
        for p, g, v in triples:
            if p.numel == 0:
                continue
            if g.numel != p.numel or (v is not None and v.numel != p.numel) or p.numel >= 2 ** 31:
                raise ValueError(f"sgd_step_: parameter {p.shape}, gradient {g.shape}")
            live.append((_addr(p), _addr(g), _addr(v) if v is not None else 0, p.numel))
        k = kernel(K.sgd_multi_inplace_kernel, momentum != 0)
        for at in range(0, len(live), M):
            part = live[at:at + M]
            blocks = [(n + 255) // 256 for *_, n in part]
            first, total = [], 0
            for b in blocks:
                first.append(total)
                total += b
            pad = M - len(part)
            launch(k, total, 256, *[q[0] for q in part], *[0] * pad, *[q[1] for q in part], *[0] * pad,
                   *[q[2] for q in part], *[0] * pad, *first, *[total] * pad, *[q[3] for q in part], *[0] * pad,
                   float(lr), float(momentum))

    ROW_MATMUL = os.environ.get("DLGRAD_HIP_ROW_MATMUL", "1") != "0"        # "0": one-row products on the MFMA tiles too
    DECODE_FUSED = os.environ.get("DLGRAD_HIP_DECODE_FUSED", "1") != "0"    # "0": cached attention as product, softmax, product
    MATMUL_PAIRS = os.environ.get("DLGRAD_HIP_MATMUL_PAIRS", "1") != "0"       # "0": the two products of a linear layer's backward as two launches
    MATMUL_PAIR_MAX_FLOP = 1 << 30        # per product: beyond it a product fills the chip by itself
    # An RMSNorm in front of a linear layer applied by the product's blocks: "1" where launches are issued one by one (a launch
    # fewer: char-GPT eager step 1.49 -> 1.33 ms), not in steps that are captured (every column block of the product
    # normalises its rows again, which costs a replayed step more than the node it saves: 0.635 -> 0.647 ms); "0" never,
    # "always" also in captured steps
    NORM_IN_PRODUCT = os.environ.get("DLGRAD_HIP_NORM_IN_PRODUCT", "1")
    CAUSAL_MASK_KNOWN = os.environ.get("DLGRAD_HIP_CAUSAL_MASK_KNOWN", "1") != "0"   # "0": the cached causal mask is read like any other mask
    CE_GRAD_ROWS = os.environ.get("DLGRAD_HIP_CE_GRAD_ROWS", "1") != "0"       # "0": the cross-entropy gradient as an element-wise launch
    # registers of the streaming attention backward held to 256 so that two blocks share a CU (312 and one block otherwise):
    # 392 -> 334 us per layer at (8, 12, 1024, 64)
    FLASH_BWD_BLOCKS_PER_CU = int(os.environ.get("DLGRAD_HIP_FLASH_BWD_BLOCKS_PER_CU", "2"))
    ATTENTION_FLASH = os.environ.get("DLGRAD_HIP_ATTENTION_FLASH", "1") != "0"   # "0": long causal attention as products and softmax launches over stored T x T tensors
    ATTENTION_FUSED = os.environ.get("DLGRAD_HIP_ATTENTION_FUSED", "1") != "0"   # "0": short causal attention as products and softmax launches too

    # ---- matmul ----------------------------------------------------------------------------------------------------------
    MATMUL_FORCE = os.environ.get("DLGRAD_HIP_MATMUL_TILE")      # e.g. "128x128": benchmarking aid
    # "1": a shape met for the first time (and large enough to matter) is timed once with every
    # plausible tile and the fastest is remembered; "0": shipped table, then the model
    MATMUL_TUNE = os.environ.get("DLGRAD_HIP_MATMUL_TUNE", "1") != "0"
    MATMUL_EXACT = os.environ.get("DLGRAD_HIP_MATMUL_EXACT", "1") != "0"    # "0": always the form of the product kernel that tests every load against the bounds
    MATMUL_SPLITK = os.environ.get("DLGRAD_HIP_MATMUL_SPLITK", "1") != "0"  # "0": never cut the k sum of a product into slices
    MATMUL_TABLE = os.environ.get("DLGRAD_HIP_MATMUL_TABLE", "1") != "0"    # "0": ignore the measured tables (model, or first-use timing, only)
    MATMUL_TUNE_MIN_FLOP = 1 << 24
    _tuned: dict | None = None
    _tuned_new: dict = {}
    _tune_warned = False                  # the first tile timing of a process says what it is doing

    MATMUL_TUNED_FILE = os.environ.get("DLGRAD_HIP_MATMUL_TUNED_FILE", os.path.join(CACHE_DIR, "matmul_tuned.json"))
    last_matmul_kernel: str | None = None      # name of the most recently launched product kernel (reported by the benchmark)

    @staticmethod
    def _tuned_path() -> str:
        return HIP.MATMUL_TUNED_FILE

    @staticmethod
    def _tuned_table() -> dict:
        """"batch,M,N,K" -> tile: the table shipped beside the kernel generators (measured on
        MI355X) overlaid with what this machine's own tuning runs have stored in the cache."""
        if HIP._tuned is None:
            table = {}
            for path in (os.path.join(os.path.dirname(K.__file__), "matmul_tuned.json"), HIP._tuned_path()) if HIP.MATMUL_TABLE else ():
                try:
                    with open(path) as f:
                        table.update({k: v for k, v in json.load(f).items() if all(HIP._valid_tile(t) for t in v.split("+"))})
                except (OSError, ValueError):
                    pass
            HIP._tuned = table
        return HIP._tuned

    @staticmethod
    def _model_tile(M: int, N: int, batch: int, Kd: int = 0) -> str:
        """Largest expected throughput = tile rate x fraction of the tile grid that is real
        output x how evenly the blocks load 256 CUs: the busiest CU runs ceil(blocks / 256) of
        them, and a CU that holds one block of a tile meant to be co-resident is given 85 %."""
        best, best_score = "64x64", -1.0
        for name, (rate, per_cu) in K.MATMUL_TILE_MODEL.items():
            bm, bn, _ = K.matmul_tile_shape(name)
            tm, tn = (M + bm - 1) // bm, (N + bn - 1) // bn
            nblk = tm * tn * batch
            rounds = -(-nblk // 256)
            fill = nblk / (256.0 * rounds)
            if rounds == 1 and per_cu > 1:
                fill *= 0.85
            score = rate * (M * N) / float(tm * bm * tn * bn) * fill
            if score > best_score * 1.0001:
                best, best_score = name, score
        small = -(-M // 64) * -(-N // 64) * batch           # blocks of the smallest 32-wide tile worth using
        if best in ("64x64", "32x32") and small <= 192 and Kd >= 32:
            # a fraction of the SIMDs busy: four times the wavefronts, 16x16 each, and as few rounds of loads as k allows
            best = "32x32m16k128" if Kd >= 128 else "32x32m16k64" if Kd >= 64 else "32x32m16"
        elif best == "64x64" and Kd >= 512 and small <= 512:
            best = "64x64k64"                       # few blocks, long K: the deep-K form of the same tile
        return best

    SPLITK_BASES = ("128x128", "128x64", "64x64k64", "64x64m16")      # tiles whose split-k forms are timed
    KGROUP_BASES = ("128x128", "128x64", "64x64", "64x64k32", "64x64k64", "32x32", "32x32m16", "64x64m16")     # tiles whose k-group forms are timed
    MATMUL_KGROUPS = os.environ.get("DLGRAD_HIP_MATMUL_KGROUPS", "1") != "0"    # "0": no product cuts k among the wavefronts of a block

    @staticmethod
    def _splitk_eligible(M: int, N: int, Kd: int, batch: int) -> bool:
        """Few output tiles (128 x 128 tiles for at most half the CUs; for all of them when k is at least 2048)
        and a k long enough to cut.  Measured on (768 x 8192)^T (8192 x 768): 60 -> 86 TFLOP/s, on the 3072-wide
        one 81 -> 100, on (128 x 2048)(2048 x 512) 11 -> 23; squares (512^3, 1024^3) gain nothing."""
        tiles = -(-M // 128) * -(-N // 128) * batch
        return HIP.MATMUL_SPLITK and ((Kd >= 512 and tiles <= 128) or (Kd >= 2048 and tiles <= 256))

    @staticmethod
    def _tile_candidates(M: int, N: int, batch: int, Kd: int = 0, split: bool = False) -> list[str]:
        """Tiles worth timing: none much larger than the output, and the two smallest only
        where the output is small enough for them to have a chance.  split: also the split-k forms of a
        few tiles, 2 to 16 slices of at least 128 k each."""
        out = []
        if split:
            for base in HIP.SPLITK_BASES:
                bm, bn, _ = K.matmul_tile_shape(base)
                if bm > max(32, 2 * M) or bn > max(32, 2 * N):
                    continue
                tiles = -(-M // bm) * -(-N // bn) * batch
                for slices in (2, 4, 8, 16):
                    if Kd // slices >= 128 and tiles * slices <= 2048 and HIP._split_plan(f"{base}/{slices}", Kd)[0] == slices:
                        out.append(f"{base}/{slices}")
            for base in HIP.KGROUP_BASES if HIP.MATMUL_KGROUPS else ():
                bm, bn, _ = K.matmul_tile_shape(base)
                if bm > max(32, 2 * M) or bn > max(32, 2 * N) or -(-M // bm) * -(-N // bn) * batch > 1024:
                    continue
                for groups in (2, 4, 8):
                    if Kd // groups >= 64 and HIP._valid_tile(f"{base}*{groups}") and HIP._group_plan(f"{base}*{groups}", Kd)[0] == groups:
                        out.append(f"{base}*{groups}")
        for name in K.MATMUL_CONFIGS:
            bm, bn, _ = K.matmul_tile_shape(name)
            if bm > max(32, 2 * M) or bn > max(32, 2 * N):
                continue
            if M * N * batch > (1 << 22 if name == "32x32" or "m16" in name else 1 << 27 if name.startswith("64x64") else 1 << 62):
                continue
            out.append(name)
        return out

    @staticmethod
    def _split_of(tile: str) -> tuple[str, int]:
        """"128x128/4" -> ("128x128", 4): the k sum cut into 4 slices, a block per (tile, slice), the partial tiles
        added up by a column-sum launch.  A plain tile name: (tile, 1).  "64x64*2" (k cut among two groups of wavefronts
        inside each block, see _groups_of) -> ("64x64", 1)."""
        base, _, sk = tile.partition("/")
        return (base.partition("*")[0], int(sk)) if sk else (base.partition("*")[0], 1)

    @staticmethod
    def _groups_of(tile: str) -> int:
        """"64x64*2" -> 2: every block has two groups of the tile's wavefronts, each with half of k (K.matmul_kernel, kgroups)."""
        _, _, g = tile.partition("*")
        return int(g) if g else 1

    @staticmethod
    def _valid_tile(tile: str) -> bool:
        try:
            base, slices = HIP._split_of(tile)
            groups = HIP._groups_of(tile)
        except ValueError:
            return False
        if base not in K.MATMUL_CONFIGS or not 1 <= slices <= 64 or (groups > 1 and (slices > 1 or groups not in (2, 3, 4, 8, 16))):
            return False
        cfg = K.MATMUL_CONFIGS[base]
        # (a group form must fit whichever operand is read transposed)
        return groups == 1 or all(K.matmul_groups_fit(*cfg[:5], ta, tb, cfg[5] if len(cfg) > 5 else 32, groups)
                                  for ta, tb in ((False, False), (True, False), (False, True)))

    @staticmethod
    def _split_plan(tile: str, Kd: int) -> tuple[int, int]:
        """(slices, kchunk) actually launched: kchunk a multiple of the tile's k step, no empty slice."""
        base, slices = HIP._split_of(tile)
        bk = K.MATMUL_CONFIGS[base][4]
        kchunk = -(-(-(-Kd // slices)) // bk) * bk
        return -(-Kd // kchunk), kchunk

    @staticmethod
    def _group_plan(tile: str, Kd: int) -> tuple[int, int]:
        """(groups, kchunk) of a k-group tile as launched: every group the same number of whole k steps (a group whose slice lies
        beyond k reads zeros); a k of fewer steps than groups were asked for gets fewer groups, down to 1 (the plain tile)."""
        base, groups = HIP._split_of(tile)[0], HIP._groups_of(tile)
        bk = K.MATMUL_CONFIGS[base][4]
        steps = -(-Kd // bk)
        if steps < groups:
            groups = max((g for g in (1, 2, 3, 4, 8, 16) if g <= steps), default=1)
        return groups, -(-steps // groups) * bk

    @staticmethod
    def _launch_matmul(tile: str, veca: bool, vecb: bool, M: int, N: int, batch: int, args: tuple,
                       ta: bool = False, tb: bool = False, tri: str = "", strided: bool = False, epi: str = "") -> None:
        if "*" in tile:
            if tri or strided or epi:
                raise ValueError(f"a k-group tile ({tile}) takes no triangular, strided or epilogue form")
            k, grid, threads = HIP._matmul_kernel(tile, veca, vecb, M, N, batch, ta, tb, Kd=args[5])
            HIP.last_matmul_kernel = kernel_names.get(id(k))
            groups, kchunk = HIP._group_plan(tile, args[5])
            launch(k, grid, threads, *args, *((kchunk,) if groups > 1 else ()))
            return
        if "/" in tile:
            if tri or strided or epi:
                raise ValueError(f"a split-k tile ({tile}) takes no triangular, strided or epilogue form")
            Kd = args[5]
            k, grid, threads = HIP._matmul_kernel(tile, veca, vecb, M, N, batch, ta, tb, Kd=Kd)
            HIP.last_matmul_kernel = kernel_names.get(id(k))
            ws = alloc(batch * grid[1] * M * N)                        # one slab per slice (handed back as soon as both launches are issued)
            launch(k, grid, threads, *args, ws.addr, HIP._split_plan(tile, Kd)[1])
            HIP._reduce_cols("sum", ws.addr, batch, grid[1], M * N, 1.0, args[2])
            return
        k, grid, threads = HIP._matmul_kernel(tile, veca, vecb, M, N, batch, ta, tb, tri, strided, epi, args[5])
        HIP.last_matmul_kernel = kernel_names.get(id(k))
        launch(k, grid, threads, *args)

    @staticmethod
    def _matmul_kernel(tile: str, veca: bool, vecb: bool, M: int, N: int, batch: int, ta: bool = False, tb: bool = False,
                       tri: str = "", strided: bool = False, epi: str = "", Kd: int = 0) -> tuple:
        """(loaded kernel, grid, threads per block) of one product (Kd: needed for a split-k tile only)."""
        base, slices = HIP._split_of(tile)
        bm, bn, threads = K.matmul_tile_shape(base)
        cfg = K.MATMUL_CONFIGS[base]                           # (WM, WN, MI, NJ, BK) and, for the 16-wide MFMA tiles, 16
        S = cfg[5] if len(cfg) > 5 else 32
        exact = HIP._whole_tiles(base, veca, vecb, M, N, Kd)
        groups = HIP._groups_of(tile)
        if groups > 1:
            groups, kchunk = HIP._group_plan(tile, Kd)
        if groups > 1:
            if tri or strided or epi or not K.matmul_groups_fit(*cfg[:5], ta, tb, S, groups):
                raise ValueError(f"tile {tile} does not fit this product (k = {Kd})")
            k = kernel(K.matmul_kernel, *cfg[:5], veca, vecb, ta, tb, "", False, "", S, False, False, exact and Kd == groups * kchunk, groups, HIP._deep_form(base))
            return k, (((M + bm - 1) // bm) * ((N + bn - 1) // bn), 1, batch), groups * threads
        if slices > 1:
            n_slices, kchunk = HIP._split_plan(tile, Kd)
            k = kernel(K.matmul_kernel, *cfg[:5], veca, vecb, ta, tb, "", False, "", S, False, True, exact and Kd % kchunk == 0, 1, HIP._deep_form(base))
            return k, (((M + bm - 1) // bm) * ((N + bn - 1) // bn), n_slices, batch), threads
        k = kernel(K.matmul_kernel, *cfg[:5], veca, vecb, ta, tb, tri, strided, epi, S, False, False, exact, 1, HIP._deep_form(base))
        return k, (((M + bm - 1) // bm) * ((N + bn - 1) // bn), 1, batch), threads

    MATMUL_DEEP = os.environ.get("DLGRAD_HIP_MATMUL_DEEP", "1") != "0"      # "0": product kernels fetch one k step ahead and store to LDS behind the MFMA run

    @staticmethod
    def _deep_form(tile: str) -> bool:
        """Whether products of this tile run the k loop that fetches two steps ahead and issues its fetches and LDS stores between
        the MFMA steps (K.matmul_kernel, deep): same bits, 4 to 17 % faster on every shape measured."""
        return HIP.MATMUL_DEEP

    @staticmethod
    def _whole_tiles(tile: str, veca: bool, vecb: bool, M: int, N: int, Kd: int) -> bool:
        """Whether a product is cut into whole tiles in every direction (and read with 16-byte loads): it then runs the form of
        the kernel whose k loop has no conditional part (K.matmul_kernel, exact) -- same bits, 2 to 12 % faster."""
        bm, bn, _ = K.matmul_tile_shape(tile)
        return bool(HIP.MATMUL_EXACT and Kd and veca and vecb and M % bm == 0 and N % bn == 0 and Kd % K.MATMUL_CONFIGS[tile][4] == 0)

    @staticmethod
    def _tune_tile(key: str, veca: bool, vecb: bool, M: int, N: int, batch: int, args: tuple,
                   ta: bool, tb: bool, tri: str = "", strided: bool = False) -> str:
        """Times every plausible tile on the real operands (the output is simply rewritten:
        all tiles produce the same bits) and stores the winner in the cache directory."""
        global launch_count
        l = lib()
        count0 = launch_count
        if not HIP._tune_warned and not COMPILE_ONLY:                # said once per process: the first step is slower, results are not
            HIP._tune_warned = True
            warnings.warn(f"dlgrad_amd: the matrix product {key} (batch,M,N,K) is in no tile table; timing every plausible tile "
                          "on its operands now, once per shape and machine (about 10 ms for mid-sized products, up to 0.5 s at "
                          "8192^3; the choice is stored in dlgrad_amd/_kcache/matmul_tuned.json; no tile changes a result bit except the split-k "
                          "forms, which add the same terms slice by slice). "
                          "DLGRAD_HIP_MATMUL_TUNE=0 switches the timing off; further shapes are timed without this message.",
                          RuntimeWarning, stacklevel=2)
        e0, e1 = l.event_create(), l.event_create()

        def sample(tile: str) -> float:
            ms, reps = 0.0, 3
            while True:
                l.event_record(e0)
                for _ in range(reps):
                    HIP._launch_matmul(tile, veca, vecb, M, N, batch, args, ta, tb, tri, strided)
                l.event_record(e1)
                l.event_sync(e1)
                ms = l.event_elapsed_ms(e0, e1) / reps
                if reps > 3 or ms > 0.1:                             # short kernels: a longer second sample
                    return ms
                reps = 20
        timed = {}
        for tile in HIP._tile_candidates(M, N, batch, args[5], key.endswith(",sk")):
            HIP._launch_matmul(tile, veca, vecb, M, N, batch, args, ta, tb, tri, strided)   # loads the code object
            if not COMPILE_ONLY:
                timed[tile] = sample(tile)
        best = min(timed, key=timed.get) if timed else None
        if best is not None:
            # tiles within 5 % of the fastest are closer than one sample can tell apart: a second sample of each, the smaller one counts
            close = [t for t in sorted(timed, key=timed.get) if timed[t] <= 1.05 * timed[best]][:4]
            if len(close) > 1:
                best = min(close, key=lambda t: min(timed[t], sample(t)))
        l.event_destroy(e0)
        l.event_destroy(e1)
        launch_count = count0
        if best is None:
            return HIP._model_tile(M, N, batch)
        HIP._tuned_table()[key] = best
        HIP._tuned_new[key] = best
        try:
            os.makedirs(os.path.dirname(HIP._tuned_path()), exist_ok=True)
            stored = {}
            if os.path.exists(HIP._tuned_path()):
                with open(HIP._tuned_path()) as f:
                    stored = json.load(f)
            stored.update(HIP._tuned_new)
            tmp = HIP._tuned_path() + f".{os.getpid()}.tmp"
            with open(tmp, "w") as f:
                json.dump(dict(sorted(stored.items())), f, indent=0)
            os.replace(tmp, HIP._tuned_path())
        except (OSError, ValueError):
            pass                                                     # a read-only tree: the choice lives for this process
        return best

    @staticmethod
    def _tile_key(M: int, N: int, Kd: int, batch: int, ta: bool = False, tb: bool = False, tri: str = "", strided: bool = False) -> str:
        """How the tile tables name a product."""
        return f"{batch},{M},{N},{Kd}" + (",tn" if ta else ",nt" if tb else "") + (f",{tri}" if tri else "") + (",ld" if strided else "")

    @staticmethod
    def _pick_tile(M: int, N: int, Kd: int, batch: int, veca: bool, vecb: bool, args: tuple,
                   ta: bool = False, tb: bool = False, tri: str = "", strided: bool = False, split_ok: bool = False) -> str:
        """split_ok: the caller can take a split-k tile (a plain product: no epilogue, structure or pitch).  Such
        products have table entries of their own (key + ",sk"), since the other forms of the same shape cannot
        use what was found for them."""
        if HIP.MATMUL_FORCE:
            return HIP.MATMUL_FORCE if split_ok else HIP._split_of(HIP.MATMUL_FORCE)[0]
        key = HIP._tile_key(M, N, Kd, batch, ta, tb, tri, strided)
        tune = HIP.MATMUL_TUNE and not capturing() and 2 * M * N * Kd * batch >= HIP.MATMUL_TUNE_MIN_FLOP
        if split_ok and not tri and not strided and HIP._splitk_eligible(M, N, Kd, batch):
            tile = HIP._tuned_table().get(key + ",sk")
            if tile is not None:
                return tile
            if tune:
                return HIP._tune_tile(key + ",sk", veca, vecb, M, N, batch, args, ta, tb)
        tile = HIP._tuned_table().get(key)
        if tile is not None:
            return HIP._split_of(tile)[0]
        if tune:
            return HIP._tune_tile(key, veca, vecb, M, N, batch, args, ta, tb, tri, strided)
        return HIP._model_tile(M, N, batch, Kd)

    @staticmethod
    @dispatcher.register(BinaryOps.MATMUL, Device.HIP)
    def matmul(x: Buffer, y: Buffer, ta: bool = False, tb: bool = False, tri: str = "", epi: str = "",
               e: Buffer | None = None, norm: tuple | None = None) -> DevicePtr:
        """x (.., M, K) @ y (.., K, N) for operands already padded to the same rank 2..4
        (buffer.py:231-243); batch dims of extent 1 broadcast through a zero stride as in
        cpu.py:519-532 and :553-559.  When y carries no batch at all the batch of x is
        folded into M: one tall GEMM instead of many small ones.
        ta: x is stored as (.., K, M) and used transposed; tb: y is stored as (.., N, K).
        tri: triangular structure of square (T x T) operands or outputs that the caller vouches
        for (K.matmul_kernel); the work it lets the kernel skip never changes a kept result.
        epi: "add" (result + e), "relu" (result where positive, else 0) or "gate" (result where e is
        positive, else 0), applied as the result is stored; e has the shape of the result.
        norm: (gain, eps[, keep]) -- the rows of x are RMS-normalised with that gain row on their way into the
        product (row_norm_fits / tile_norm_fits say where this is provided): the RMSNorm launch in front of a
        linear layer disappears, the values are those of the two launches.  With keep the normalised rows and
        the per-row 1 / rms are returned as well: (result, normalised x, rinv)."""
        xa, ya = x.ptr.addr, y.ptr.addr
        ea = 0 if e is None or e.ptr.__class__ is HostScalar else e.ptr.addr
        if norm is not None:
            gain, eps, keep = norm[0], float(norm[1]), len(norm) > 2 and bool(norm[2])
            if epi not in ("", "add", "relu", "gate") or ta or tri:
                raise ValueError(f"a normalising product does not take epi={epi!r}, ta={ta}, tri={tri!r}")
            if not keep and tb and HIP.row_norm_fits(x, y, gain):
                N, Kd = y.shape[-2:]
                if epi in ("add", "gate") and (not ea or e.numel != N or ea & 15):
                    raise ValueError(f"epilogue {epi!r} of a normalising product needs an aligned operand of {N} elements")
                out = alloc(N)
                k = kernel(K.row_matmul_nt_kernel, epi, K.rmsnorm_plan(Kd, 4))
                launch(k, (N + 3) // 4, 256, xa, ya, out.addr, ea, N, Kd, _addr(gain), eps)
                return out
            if not HIP.tile_norm_fits(x, y, gain, tb):
                raise ValueError(f"a normalising product is not provided for {x.shape} x {y.shape}")
            Kd = x.shape[-1]
            M, N = x.numel // Kd, y.shape[-2] if tb else y.shape[-1]
            if epi in ("add", "gate") and (not ea or e.numel != M * N):
                raise ValueError(f"epilogue {epi!r} needs an operand shaped like the result ({M * N} elements)")
            out = alloc(M * N)
            yn, rinv = (alloc(M * Kd), alloc(M)) if keep else (None, None)
            vecb = (Kd if tb else N) % 4 == 0 and not (ya & 15)
            if epi and e is not None and (ea & 15 or N % 4):
                vecb = False                                   # the epilogue reads e as it writes the result
            tile = HIP.MATMUL_FORCE if K.MATMUL_CONFIGS.get(HIP.MATMUL_FORCE, (0,) * 5)[4] >= Kd else \
                ("64x64m16k128" if N >= 256 and M >= 64 else "32x32m16k128")       # tiles whose k step holds a whole row
            cfg = K.MATMUL_CONFIGS[tile]
            bm, bn, threads = K.matmul_tile_shape(tile)
            k = kernel(K.matmul_kernel, *cfg[:5], True, vecb, False, tb, "", False, epi, cfg[5] if len(cfg) > 5 else 32, True)
            HIP.last_matmul_kernel = kernel_names.get(id(k))
            tail = ((ea or out.addr,) if epi else ()) + (_addr(gain), eps, yn.addr if keep else 0, rinv.addr if keep else 0)
            launch(k, (((M + bm - 1) // bm) * ((N + bn - 1) // bn), 1, 1), threads, xa, ya, out.addr, M, N, Kd, 1, 0, 0, 0, 0, *tail)
            return (out, yn, rinv) if keep else out
        key = (x.shape, y.shape, ta, tb, tri, epi, None if e is None else e.shape, xa & 15, ya & 15, ea & 15,
               HIP.MATMUL_FORCE, HIP.ROW_MATMUL, HIP.MATMUL_SPLITK, HIP.MATMUL_EXACT, HIP.MATMUL_KGROUPS, HIP.MATMUL_DEEP)
        plan = _matmul_plans.get(key)
        if plan is not None:                                   # a shape seen before: pack the addresses and go
            k, grid, threads, tail, out_numel, e_at, name = plan
            if e_at == 3:                                      # a split-k tile: a workspace and a second launch
                out = alloc(out_numel)
                HIP._launch_matmul(k, *grid, (xa, ya, out.addr, *tail), *threads)
                return out
            if e_at == 0:                                      # (x, y, out, sizes and strides)
                HIP.last_matmul_kernel = name
                return launch_out(k, grid, threads, 16, out_numel, xa, ya, 0, *tail)
            if e_at == 1:                                      # the same with the epilogue's operand at the end
                HIP.last_matmul_kernel = name
                return launch_out(k, grid, threads, 16, out_numel, xa, ya, 0, *tail, ea)
            return launch_out(k, grid, threads, 16, out_numel, xa, ya, 0, ea, *tail)        # the single-row kernel: (x, W, out, e, N, K)
        assert x.ndim == y.ndim and 2 <= x.ndim <= 4 and not (ta and tb)
        (Kd, M) = x.shape[-2:] if ta else x.shape[-2:][::-1]
        (N, Ky) = y.shape[-2:] if tb else y.shape[-2:][::-1]
        assert Ky == Kd, f"inner dims differ: {x.shape} {y.shape} ta={ta} tb={tb}"
        xb = (1,) * (4 - x.ndim) + tuple(x.shape[:-2])
        yb = (1,) * (4 - y.ndim) + tuple(y.shape[:-2])
        B0, B1 = max(xb[0], yb[0]), max(xb[1], yb[1])
        out_numel = B0 * B1 * M * N
        out = alloc(out_numel)
        if epi:
            if epi not in ("add", "relu", "gate", "bias") or tri:
                raise ValueError(f"epilogue {epi!r} with tri={tri!r} is not provided")
            if epi == "bias":
                if e is None or e.is_host_scalar or e.numel != N:
                    raise ValueError(f"epilogue 'bias' needs a row of {N} values")
            elif epi != "relu" and (e is None or e.is_host_scalar or e.numel != B0 * B1 * M * N):
                raise ValueError(f"epilogue {epi!r} needs an operand shaped like the result ({B0 * B1 * M * N} elements)")
        if B0 * B1 * M * N == 0:
            return out
        if Kd == 0:                                            # an empty sum: zeros, plus e for "add"
            if epi == "add":
                lib().d2d(out.addr, _addr(e), 4 * B0 * B1 * M * N)
            elif epi == "bias":
                for r in range(B0 * B1 * M):
                    lib().d2d(out.addr + 4 * r * N, _addr(e), 4 * N)
            else:
                lib().fill_f32(out.addr, 0.0, B0 * B1 * M * N)
            return out
        if tri:
            square = {"out_lower": M == N, "a_lower": not ta and M == Kd, "at_lower": ta and M == Kd}.get(tri)
            if not square:
                raise ValueError(f"tri={tri!r} does not fit {x.shape} x {y.shape} (ta={ta}, tb={tb})")
        if yb == (1, 1) and not ta and not tri:
            M, nbc, batch = xb[0] * xb[1] * M, 1, 1
            sa = sb = (0, 0)
        else:
            nbc, batch = B1, B0 * B1
            sa = (xb[1] * M * Kd if xb[0] > 1 else 0, M * Kd if xb[1] > 1 else 0)
            sb = (yb[1] * Kd * N if yb[0] > 1 else 0, Kd * N if yb[1] > 1 else 0)
        if (M == 1 and batch == 1 and tb and not ta and not tri and HIP.ROW_MATMUL and not HIP.MATMUL_FORCE and Kd % 4 == 0
                and not ((_addr(x) | _addr(y)) & 15) and (e is None or not e.is_host_scalar)):
            # one row against a transposed matrix (a linear layer while decoding): a wavefront per output
            k = kernel(K.row_matmul_nt_kernel, "add" if epi == "bias" else epi)      # (for a single row the bias is the residual)
            launch(k, (N + 3) // 4, 256, _addr(x), _addr(y), out.addr, _addr(e) if e is not None else 0, N, Kd)
            _matmul_plans[key] = (k, ((N + 3) // 4, 1, 1), (256, 1, 1), (N, Kd), N, 2, None)
            return out
        if batch > 65535:
            raise ValueError(f"{batch} batches exceed the grid limit")
        if max(M * Kd, Kd * N, M * N) >= 2 ** 31:
            raise ValueError("matrix too large for 32-bit indexing")
        veca = (M if ta else Kd) % 4 == 0 and _addr(x) % 16 == 0
        vecb = (Kd if tb else N) % 4 == 0 and _addr(y) % 16 == 0 and out.addr % 16 == 0
        if epi and e is not None and (_addr(e) % 16 or N % 4):
            vecb = False                                       # the epilogue reads e as it writes the result
        args = (_addr(x), _addr(y), out.addr, M, N, Kd, nbc, *sa, *sb)
        tile = HIP._pick_tile(M, N, Kd, batch, veca, vecb, args, ta, tb, tri, split_ok=not epi and not tri)
        if epi:
            HIP._launch_matmul(tile, veca, vecb, M, N, batch, (*args, out.addr if e is None else _addr(e)), ta, tb, "", False, epi)
        else:
            HIP._launch_matmul(tile, veca, vecb, M, N, batch, args, ta, tb, tri)
        if not capturing():                                    # (while capturing, a shape met for the first time is not timed)
            if "/" in tile:
                _matmul_plans[key] = (tile, (veca, vecb, M, N, batch), (ta, tb), args[3:], out_numel, 3, HIP.last_matmul_kernel)
            elif "*" in tile:
                k, grid, threads = HIP._matmul_kernel(tile, veca, vecb, M, N, batch, ta, tb, Kd=Kd)
                groups, kchunk = HIP._group_plan(tile, Kd)
                _matmul_plans[key] = (k, grid, threads, (*args[3:], *((kchunk,) if groups > 1 else ())), out_numel, 0, HIP.last_matmul_kernel)
            else:
                k, grid, threads = HIP._matmul_kernel(tile, veca, vecb, M, N, batch, ta, tb, "" if epi else tri, False, epi, Kd)
                _matmul_plans[key] = (k, grid, threads, args[3:], out_numel, 1 if epi else 0, HIP.last_matmul_kernel)
        return out

    @staticmethod
    def _pair_part(x: Buffer, y: Buffer, ta: bool, tb: bool, epi: str, e: Buffer | None):
        """Sizes and strides of one product of a pair as HIP.matmul lays it out -- (M, N, K, nbc, batch, sa, sb,
        out_numel) -- or None where that product takes one of HIP.matmul's special routes or is too
        large to gain from company."""
        if x.ndim != y.ndim or not 2 <= x.ndim <= 4 or (ta and tb):
            return None
        (Kd, M) = x.shape[-2:] if ta else x.shape[-2:][::-1]
        (N, Ky) = y.shape[-2:] if tb else y.shape[-2:][::-1]
        xb = (1,) * (4 - x.ndim) + tuple(x.shape[:-2])
        yb = (1,) * (4 - y.ndim) + tuple(y.shape[:-2])
        B0, B1 = max(xb[0], yb[0]), max(xb[1], yb[1])
        out_numel = B0 * B1 * M * N
        if Ky != Kd or Kd == 0 or out_numel == 0:
            return None
        if epi and (epi not in ("add", "relu", "gate") or (epi != "relu" and (e is None or e.is_host_scalar or e.numel != out_numel))):
            return None
        if yb == (1, 1) and not ta:
            M, nbc, batch = xb[0] * xb[1] * M, 1, 1
            sa = sb = (0, 0)
        else:
            nbc, batch = B1, B0 * B1
            sa = (xb[1] * M * Kd if xb[0] > 1 else 0, M * Kd if xb[1] > 1 else 0)
            sb = (yb[1] * Kd * N if yb[0] > 1 else 0, Kd * N if yb[1] > 1 else 0)
        if (M == 1 and batch == 1 and tb) or batch > 65535 or max(M * Kd, Kd * N, M * N) >= 2 ** 31:
            return None
        if 2 * M * N * Kd * batch > HIP.MATMUL_PAIR_MAX_FLOP:
            return None
        return M, N, Kd, nbc, batch, sa, sb, out_numel

    @staticmethod
    @dispatcher.register(CustomOps.MATMUL_PAIR, Device.HIP)
    def matmul_pair(first: tuple, second: tuple) -> tuple[DevicePtr, DevicePtr]:
        """Two independent products (x, y, ta, tb, epi, e), operands prepared as for HIP.matmul, as one launch
        (K.matmul_pair_kernel): the backward of a linear layer needs dX = G W and dW = G^T X, which share
        an input and nothing else, and either alone leaves most of the chip idle while its short k loop
        runs.  Each product keeps the tile it would have on its own and its bits.  Large products, and the
        shapes HIP.matmul treats specially, go out as two launches."""
        specs = (first, second)
        addrs = tuple((x.ptr.addr, y.ptr.addr, 0 if e is None or e.ptr.__class__ is HostScalar else e.ptr.addr)
                      for x, y, _, _, _, e in specs)
        key = tuple((x.shape, y.shape, ta, tb, epi, None if e is None else e.shape, a[0] & 15, a[1] & 15, a[2] & 15)
                    for (x, y, ta, tb, epi, e), a in zip(specs, addrs)) + (HIP.MATMUL_FORCE, HIP.MATMUL_EXACT, HIP.MATMUL_DEEP)
        plan = _pair_plans.get(key)
        if plan is None:
            parts = [HIP._pair_part(*sp) for sp in specs]
            if None in parts:
                plan = _pair_plans[key] = False
            elif capturing():                             # a pair met for the first time while capturing: tiles are not timed now
                plan = False
            else:
                cfgs, tails, grids, numels, has_e = [], [], [], [], []
                # a pair that has been timed as a pair (the table's "pair:" entries) takes the two tiles that were fastest together,
                # which need not be the ones that are fastest alone
                pair_key = "pair:" + "|".join(HIP._tile_key(M, N, Kd, batch, ta, tb) + (f",{epi}" if epi else "")
                                              for (_, _, ta, tb, epi, _), (M, N, Kd, _, batch, _, _, _) in zip(specs, parts))
                together = None if HIP.MATMUL_FORCE else HIP._tuned_table().get(pair_key)
                together = together.split("+") if together else None
                for (x, y, ta, tb, epi, e), a, (M, N, Kd, nbc, batch, sa, sb, out_numel) in zip(specs, addrs, parts):
                    veca = (M if ta else Kd) % 4 == 0 and a[0] % 16 == 0
                    vecb = (Kd if tb else N) % 4 == 0 and a[1] % 16 == 0
                    if epi and e is not None and (a[2] % 16 or N % 4):
                        vecb = False
                    probe = alloc(out_numel)              # tiles are timed on a result of the real size
                    tile = together[len(cfgs)] if together else HIP._pick_tile(
                        M, N, Kd, batch, veca, vecb, (a[0], a[1], probe.addr, M, N, Kd, nbc, *sa, *sb), ta, tb)
                    bm, bn, _ = K.matmul_tile_shape(tile)
                    cfg = K.MATMUL_CONFIGS[tile]
                    cfgs.append((*cfg[:5], veca, vecb, ta, tb, "", False, epi, cfg[5] if len(cfg) > 5 else 32,
                                 HIP._whole_tiles(tile, veca, vecb, M, N, Kd), HIP._deep_form(tile)))
                    tails.append((M, N, Kd, nbc, *sa, *sb))
                    grids.append((((M + bm - 1) // bm) * ((N + bn - 1) // bn), batch))
                    numels.append(out_numel)
                    has_e.append(bool(epi))
                k = kernel(K.matmul_pair_kernel, cfgs[0], cfgs[1])
                nb0, nb1 = grids[0][0] * grids[0][1], grids[1][0] * grids[1][1]
                plan = _pair_plans[key] = (k, nb0 + nb1, max(64 * c[0] * c[1] for c in cfgs), tails, numels, has_e,
                                           (nb0, grids[0][0], grids[1][0]), kernel_names.get(id(k)))
        if not plan:
            return tuple(HIP.matmul(x, y, ta=ta, tb=tb, epi=epi, e=e) for x, y, ta, tb, epi, e in specs)
        k, nblk, threads, tails, numels, has_e, tail, name = plan
        outs = (alloc(numels[0]), alloc(numels[1]))
        args = []
        for a, out, t, he in zip(addrs, outs, tails, has_e):
            args += [a[0], a[1], out.addr, *t]
            if he:
                args.append(a[2] or out.addr)             # "relu" looks at the result only
        HIP.last_matmul_kernel = name
        launch(k, nblk, threads, *args, *tail)
        return outs

    @staticmethod
    def row_norm_fits(x: Buffer, w: Buffer, gain: Buffer) -> bool:
        """Whether the single-row product kernel takes x (one row of K) against w stored (N, K) and can RMS-normalise x
        with the gain row on the way: the row fits a wavefront's registers and everything is read 16 bytes at a time."""
        Kd = x.shape[-1] if x.ndim else 0
        return (HIP.ROW_MATMUL and not HIP.MATMUL_FORCE and x.numel == Kd and Kd > 0 and Kd % 4 == 0 and w.ndim >= 2 and w.numel == w.shape[-2] * Kd
                and w.shape[-1] == Kd and gain.numel == Kd and 0 < K.rmsnorm_plan(Kd, 4) <= 4
                and not ((_addr(x) | _addr(w) | _addr(gain)) & 15))

    @staticmethod
    def tile_norm_fits(x: Buffer, w: Buffer, gain: Buffer, tb: bool = True) -> bool:
        """Whether the tile product can RMS-normalise the rows of x (.., K) on their way: K fits one k step of the
        deepest tiles (so a block's tile of x holds whole rows), w is a single matrix -- (N, K) if tb else (K, N) --
        and x and the gain row are read 16 bytes at a time."""
        Kd = x.shape[-1] if x.ndim else 0
        return (0 < Kd <= 128 and Kd % 4 == 0 and x.numel >= Kd and x.numel < 2 ** 31 and w.ndim >= 2 and w.numel == w.shape[-1] * w.shape[-2]
                and (w.shape[-1] if tb else w.shape[-2]) == Kd and gain.numel == Kd and w.numel < 2 ** 31
                and (x.numel // Kd) * (w.numel // Kd) < 2 ** 31 and not ((_addr(x) | _addr(gain)) & 15))

    @staticmethod
    @dispatcher.register(CustomOps.MATMUL_NT, Device.HIP)
    def matmul_nt(x: Buffer, y: Buffer, tri: str = "", epi: str = "", e: Buffer | None = None, norm: tuple | None = None) -> DevicePtr:
        """x (.., M, K) times the transpose of y (.., N, K), read in place."""
        return HIP.matmul(x, y, tb=True, tri=tri, epi=epi, e=e, norm=norm)

    @staticmethod
    @dispatcher.register(CustomOps.MATMUL_TN, Device.HIP)
    def matmul_tn(x: Buffer, y: Buffer, tri: str = "") -> DevicePtr:
        """The transpose of x (.., K, M), read in place, times y (.., K, N)."""
        return HIP.matmul(x, y, ta=True, tri=tri)

    @staticmethod
    def _gemm_strided(A: tuple, B: tuple, C: tuple, M: int, N: int, Kd: int, B0: int, B1: int,
                      ta: bool = False, tb: bool = False, tri: str = "", rows_group: int = 0) -> None:
        """C[b0, b1] = op(A[b0, b1]) . op(B[b0, b1]) for matrices cut out of larger tensors: every
        operand is (address, row pitch, stride of b0, stride of b1) in floats.  Same kernel, same
        order of additions as the contiguous product of the same logical matrices.
        rows_group: with tri, the structured operand holds defined values only inside aligned groups of that
        many rows along the diagonal, so the tile's rows must divide it."""
        (aa, lda, sa0, sa1), (ba, ldb, sb0, sb1), (ca, ldc, sc0, sc1) = A, B, C
        key = (A[1:], B[1:], C[1:], M, N, Kd, B0, B1, ta, tb, tri, aa & 15, ba & 15, ca & 15, HIP.MATMUL_FORCE, rows_group, HIP.MATMUL_EXACT, HIP.MATMUL_DEEP)
        plan = _gemm_plans.get(key)
        if plan is not None:
            k, grid, threads, tail = plan
            launch(k, grid, threads, aa, ba, ca, *tail)
            return
        if B0 * B1 > 65535 or max(lda * max(M, Kd), ldb * max(N, Kd), ldc * M) >= 2 ** 31:
            raise ValueError("strided product too large for the grid or for 32-bit indexing")
        al4 = lambda addr, *v: addr % 16 == 0 and all(x % 4 == 0 for x in v)     # noqa: E731
        veca = (M if ta else Kd) % 4 == 0 and al4(aa, lda, sa0, sa1)
        vecb = (Kd if tb else N) % 4 == 0 and al4(ba, ldb, sb0, sb1) and al4(ca, ldc, sc0, sc1)
        args = (aa, ba, ca, M, N, Kd, B1, sa0, sa1, sb0, sb1, lda, ldb, ldc, sc0, sc1)
        batch = B0 * B1
        tile = HIP._pick_tile(M, N, Kd, batch, veca, vecb, args, ta, tb, tri, True)
        if rows_group and rows_group % K.matmul_tile_shape(tile)[0]:
            tile = "64x64k64"                                  # the caller's operand is only defined in aligned groups of rows_group rows
        HIP._launch_matmul(tile, veca, vecb, M, N, batch, args, ta, tb, tri, True)
        if not capturing():
            _gemm_plans[key] = (*HIP._matmul_kernel(tile, veca, vecb, M, N, batch, ta, tb, tri, True, "", Kd), args[3:])

    @staticmethod
    def _heads(addr: int, T: int, C: int, d: int) -> tuple:
        """The (T x d) head matrices inside a (B, T, C) tensor: pitch C, batch strides T*C and d."""
        return (addr, C, T * C, d)

    @staticmethod
    def _attention_fits(T: int, d: int, heads: int, read_addrs: tuple, read_pitches: tuple) -> bool:
        """Whether the one-block-per-head attention kernels take the case: the head fits their LDS tiles
        and every tensor they read with 16-byte loads is laid out for that."""
        return (HIP.ATTENTION_FUSED and 0 < T <= K.ATTN_SMALL_T and 0 < d <= K.ATTN_SMALL_D and d % 4 == 0
                and 0 < heads < 2 ** 29 and not any(a & 15 for a in read_addrs) and not any(q & 3 for q in read_pitches))

    @staticmethod
    def _flash_fits(T: int, d: int, heads: int, addrs: tuple, pitches: tuple) -> bool:
        """Whether the streaming attention kernels take the case (any T; heads of up to 64 columns, 16-byte accesses)."""
        return (HIP.ATTENTION_FLASH and T > 0 and 0 < d <= K.ATTN_FLASH_D and d % 4 == 0 and T < 2 ** 20
                and 0 < heads * ((T + 127) // 128) < 2 ** 31 and not any(a & 15 for a in addrs) and not any(q & 3 for q in pitches))

    @staticmethod
    def _attend(qa: int, ka: int, va: int, pitch: int, ya: int, y_pitch: int, Bn: int, T: int, n_head: int, d: int,
                scale: float) -> DevicePtr:
        """Causal attention over heads that lie at addresses qa, ka, va with row pitch `pitch` (batch
        stride T * pitch, head stride d); the context goes to ya with pitch y_pitch.  Returns what the
        backward pass needs besides its inputs: the probabilities (Bn, n_head, T, T), or -- from the
        streaming kernels, which never store them -- the log-sum-exp of every score row (Bn, n_head, T)."""
        from dlgrad_amd.ops import causal_mask
        if HIP._attention_fits(T, d, Bn * n_head, (qa, ka, va), (pitch,)):
            # one block per (sequence, head, 32 rows): scores, softmax and context without leaving the chip
            p = alloc(Bn * n_head * T * T)
            nt = (T + 31) // 32
            launch(kernel(K.attention_small_kernel, "fwd"), Bn * n_head * nt, 512, qa, ka, va, ya, p.addr, T, d, pitch, y_pitch,
                   n_head, nt, float(scale))
            return p
        if HIP._flash_fits(T, d, Bn * n_head, (qa, ka, va, ya), (pitch, y_pitch)):
            # one block per (sequence, head, 128 queries): keys and values stream past, online softmax, no T x T tensor
            lse = alloc(Bn * n_head * T)
            nq = (T + 127) // 128
            launch(kernel(K.attention_flash_kernel, "fwd", 32 if d <= 32 else 64), Bn * n_head * nq, 256, qa, ka, va, ya, lse.addr,
                   T, d, pitch, y_pitch, n_head, nq, float(scale))
            return lse
        raw = alloc(Bn * n_head * T * T)
        dense = lambda addr: (addr, T, n_head * T * T, T * T)                       # noqa: E731
        HIP._gemm_strided(HIP._heads(qa, T, pitch, d), HIP._heads(ka, T, pitch, d), dense(raw.addr), T, T, d, Bn, n_head,
                          tb=True, tri="out_lower")
        p = HIP.masked_softmax(Buffer(raw, (Bn, n_head, T, T), Device.HIP), causal_mask(T, Device.HIP), scale)
        HIP._gemm_strided(dense(p.addr), HIP._heads(va, T, pitch, d), HIP._heads(ya, T, y_pitch, d),
                          T, d, T, Bn, n_head, tri="a_lower")
        return p

    @staticmethod
    def _attend_bwd(qa: int, ka: int, va: int, pitch: int, p: Buffer, dya: int, dy_pitch: int, dqa: int, dka: int,
                    dva: int, g_pitch: int, Bn: int, T: int, n_head: int, d: int, scale: float, ya: int | None = None) -> None:
        """Gradients of _attend, written to dqa, dka, dva with row pitch g_pitch.  ya: the context that
        _attend wrote, laid out like dy, if the caller kept it (the one-launch kernel wants it)."""
        from dlgrad_amd.ops import causal_mask
        if ya is not None and HIP._attention_fits(T, d, Bn * n_head, (qa, ka, va, dya, ya), (pitch, dy_pitch)):
            nt = (T + 31) // 32
            launch(kernel(K.attention_small_kernel, "bwd"), Bn * n_head * nt, 512, qa, ka, va, _addr(p), ya, dya, dqa, dka, dva,
                   T, d, pitch, dy_pitch, g_pitch, n_head, nt, float(scale))
            return
        if p.numel == Bn * n_head * T and (T > 1 or HIP._flash_fits(T, d, Bn * n_head, (qa, ka, va), (pitch,))):
            # p is the log-sum-exp per score row (the streaming forward): probabilities are recomputed tile by tile
            if ya is None or not HIP._flash_fits(T, d, Bn * n_head, (qa, ka, va, dya, ya, dka, dva), (pitch, dy_pitch, g_pitch)):
                raise ValueError("the streaming attention backward needs the forward context and 16-byte aligned heads")
            delta = alloc(Bn * n_head * T)
            rows = Bn * T * n_head
            launch(kernel(K.attention_flash_kernel, "delta", 32), (rows + 15) // 16, 256, dya, ya, delta.addr, rows, T, d, dy_pitch, n_head)
            ds = alloc(Bn * n_head * T * T)
            nk = (T + 127) // 128
            launch(kernel(K.attention_flash_kernel, "bwd", 32 if d <= 32 else 64, HIP.FLASH_BWD_BLOCKS_PER_CU), Bn * n_head * nk, 256, qa, ka, va, dya, _addr(p),
                   delta.addr, ds.addr, dka, dva, T, d, pitch, dy_pitch, g_pitch, n_head, nk, float(scale))
            HIP._gemm_strided((ds.addr, T, n_head * T * T, T * T), HIP._heads(ka, T, pitch, d), HIP._heads(dqa, T, g_pitch, d),
                              T, d, T, Bn, n_head, tri="a_lower", rows_group=256)
            return
        dense = lambda addr: (addr, T, n_head * T * T, T * T)                       # noqa: E731
        dp = alloc(p.numel)
        HIP._gemm_strided(HIP._heads(dya, T, dy_pitch, d), HIP._heads(va, T, pitch, d), dense(dp.addr), T, T, d, Bn, n_head,
                          tb=True, tri="out_lower")
        HIP._gemm_strided(dense(_addr(p)), HIP._heads(dya, T, dy_pitch, d), HIP._heads(dva, T, g_pitch, d),
                          T, d, T, Bn, n_head, ta=True, tri="at_lower")
        ds = HIP.masked_softmax_bwd(p, Buffer(dp, p.shape, Device.HIP), causal_mask(T, Device.HIP), scale)
        HIP._gemm_strided(dense(ds.addr), HIP._heads(ka, T, pitch, d), HIP._heads(dqa, T, g_pitch, d),
                          T, d, T, Bn, n_head, tri="a_lower")
        HIP._gemm_strided(dense(ds.addr), HIP._heads(qa, T, pitch, d), HIP._heads(dka, T, g_pitch, d),
                          T, d, T, Bn, n_head, ta=True, tri="at_lower")

    @staticmethod
    @dispatcher.register(CustomOps.CAUSAL_ATTENTION_QKV, Device.HIP)
    def causal_attention_qkv(qkv: Buffer, n_head: int, scale: float) -> tuple[DevicePtr, DevicePtr]:
        """causal_attention for q, k and v interleaved per position as one (B, T, 3C) tensor -- the
        output of a single projection with the three weight matrices stacked: the heads are read
        with row pitch 3C.  Returns (y (B, T, C), p)."""
        Bn, T, C3 = qkv.shape
        C = C3 // 3
        a = _addr(qkv)
        y = alloc(Bn * T * C)
        p = HIP._attend(a, a + 4 * C, a + 8 * C, C3, y.addr, C, Bn, T, n_head, C // n_head, scale)
        return y, p

    @staticmethod
    @dispatcher.register(CustomOps.CAUSAL_ATTENTION_QKV_BWD, Device.HIP)
    def causal_attention_qkv_bwd(qkv: Buffer, p: Buffer, dy: Buffer, n_head: int, scale: float, y: Buffer | None = None) -> DevicePtr:
        """Gradient of causal_attention_qkv with respect to qkv, in the same (B, T, 3C) layout.  y: the
        context of the forward pass, if kept."""
        Bn, T, C3 = qkv.shape
        C = C3 // 3
        a = _addr(qkv)
        g = alloc(Bn * T * C3)
        HIP._attend_bwd(a, a + 4 * C, a + 8 * C, C3, p, _addr(dy), C, g.addr, g.addr + 4 * C, g.addr + 8 * C, C3,
                        Bn, T, n_head, C // n_head, scale, None if y is None else _addr(y))
        return g

    @staticmethod
    @dispatcher.register(CustomOps.CAUSAL_ATTENTION, Device.HIP)
    def causal_attention(q: Buffer, k: Buffer, v: Buffer, n_head: int, scale: float) -> tuple[DevicePtr, DevicePtr]:
        """Causal attention for q, k, v given as (B, T, C) projections with C = n_head * d: the heads are
        read where they lie and the context is written straight into (B, T, C), so the four head
        transposes of examples/gpt.py:46-48,57 never materialise.  Returns (y, p) with the
        probabilities p (B, n_head, T, T) kept for the backward pass.  The products and the
        softmax are the kernels of the op-by-op chain, with the causal structure known."""
        Bn, T, C = q.shape
        y = alloc(Bn * T * C)
        p = HIP._attend(_addr(q), _addr(k), _addr(v), C, y.addr, C, Bn, T, n_head, C // n_head, scale)
        return y, p

    @staticmethod
    @dispatcher.register(CustomOps.CACHED_ATTENTION, Device.HIP)
    def cached_attention(q: Buffer, k_store: Buffer, v_store: Buffer, n: int, n_head: int, scale: float,
                         hidden: Buffer | None = None) -> DevicePtr:
        """One new position per sequence, q (B, 1, C), attending to the first n rows of key/value
        stores laid out (block, B, C): softmax(q k^T * scale) v per head, the heads read where they
        lie in q and in the stores and the context written as (B, 1, C).  `hidden` (.., n) marks rows
        to leave out (-inf before the softmax).  Inference only."""
        Bn, _, C = q.shape
        d = C // n_head
        if q.shape[1] != 1 or C % n_head or n < 1:
            raise ValueError(f"cached_attention: q {q.shape} is not one position of {n_head} heads, or n = {n}")
        for store in (k_store, v_store):
            if store.ndim != 3 or store.shape[1:] != (Bn, C) or store.shape[0] < n:
                raise ValueError(f"cached_attention: a store of shape {store.shape} does not hold {n} rows of ({Bn}, {C})")
        if HIP.DECODE_FUSED and 0 < n <= K.DECODE_ATTENTION_MAX_N and d <= K.DECODE_ATTENTION_MAX_D and Bn * n_head < 2 ** 31:
            # one wavefront per (sequence, head) does scores, softmax and context in one launch
            if hidden is not None and hidden.numel < n:
                raise ValueError(f"cached_attention: hidden {hidden.shape} is shorter than {n} positions")
            y = alloc(Bn * C)
            addrs = (_addr(q), _addr(k_store), _addr(v_store))
            vec = 4 if (d in (4, 8, 16, 32, 64) and C % 4 == 0 and not any(a & 15 for a in addrs + (y.addr,))) else 1
            npl = next(v for v in (2, 4, 8, 16) if 64 * v >= n)
            launch(kernel(K.decode_attention_kernel, npl, hidden is not None, vec), Bn * n_head, 64, *addrs,
                   _addr(hidden) if hidden is not None else 0, y.addr, n, C, d, Bn * C, n_head, float(scale))
            return y
        store_heads = lambda buf: (_addr(buf), Bn * C, C, d)                        # noqa: E731  rows = positions
        one_row = lambda addr: (addr, C, C, d)                                        # noqa: E731  (B, 1, C)
        s = alloc(Bn * n_head * n)
        dense = (s.addr, n, n_head * n, n)
        HIP._gemm_strided(one_row(_addr(q)), store_heads(k_store), dense, 1, n, d, Bn, n_head, tb=True)
        if hidden is None:                                   # nothing to leave out: a mask of zeros
            if _graph_depth:
                zeros = alloc(n, zero=True)                      # an arena's memory must not outlive it
            else:
                zeros = _state.get("zeros")
                if zeros is None or zeros.nbytes < 4 * n:
                    zeros = _state["zeros"] = alloc(max(n, 1024), zero=True)
            hidden = Buffer(zeros, (n,), Device.HIP)
        p = HIP.masked_softmax(Buffer(s, (Bn, n_head, 1, n), Device.HIP), hidden, scale)
        y = alloc(Bn * C)
        HIP._gemm_strided((p.addr, n, n_head * n, n), store_heads(v_store), one_row(y.addr), 1, d, n, Bn, n_head)
        return y

    @staticmethod
    @dispatcher.register(CustomOps.CAUSAL_ATTENTION_BWD, Device.HIP)
    def causal_attention_bwd(q: Buffer, k: Buffer, v: Buffer, p: Buffer, dy: Buffer, n_head: int,
                             scale: float, y: Buffer | None = None) -> tuple[DevicePtr, DevicePtr, DevicePtr]:
        """Gradients of causal_attention with respect to the (B, T, C) projections, written in that layout."""
        Bn, T, C = q.shape
        dq, dk, dv = alloc(Bn * T * C), alloc(Bn * T * C), alloc(Bn * T * C)
        HIP._attend_bwd(_addr(q), _addr(k), _addr(v), C, p, _addr(dy), C, dq.addr, dk.addr, dv.addr, C,
                        Bn, T, n_head, C // n_head, scale, None if y is None else _addr(y))
        return dq, dk, dv
