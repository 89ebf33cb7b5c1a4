"""Loads libdlgrad_hip.so and exposes include/dlgrad_hip.h as Python calls.

The reference talks to its C kernels through cffi (dlgrad/runtime/cpu.py:49,
:69-78).  cffi is used here too when it is importable; otherwise the stdlib
`ctypes` binds the same symbols, so the backend also loads on machines that
have no cffi wheel.  Both paths present one small object, `HipLib`, whose
methods take and return plain ints / bytes; nothing above this file knows which
binding is active.  A missing library is an ImportError-like RuntimeError: the
hip runtime never falls back to another device.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("DLGRAD_HIP_LIB", os.path.join(_HERE, "libdlgrad_hip.so"))
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "dlgrad_hip.h")

# name -> (restype, argtypes) for the ctypes binding; kept in the order of the header
_c = ctypes
_SIGS = {
    "dlg_hip_init": (_c.c_int, [_c.c_int]),
    "dlg_hip_device_count": (_c.c_int, [_c.POINTER(_c.c_int)]),
    "dlg_hip_props": (_c.c_int, [_c.c_void_p]),
    "dlg_hip_shutdown": (_c.c_int, []),
    "dlg_hip_alloc": (_c.c_int, [_c.c_size_t, _c.POINTER(_c.c_void_p)]),
    "dlg_hip_alloc_zero": (_c.c_int, [_c.c_size_t, _c.POINTER(_c.c_void_p)]),
    "dlg_hip_fill_f32": (_c.c_int, [_c.c_void_p, _c.c_float, _c.c_size_t]),
    "dlg_hip_free": (_c.c_int, [_c.c_void_p]),
    "dlg_hip_pool_stats": (_c.c_int, [_c.POINTER(_c.c_uint64)] * 3),
    "dlg_hip_pool_trim": (_c.c_int, []),
    "dlg_hip_h2d": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_size_t]),
    "dlg_hip_d2h": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_size_t]),
    "dlg_hip_d2d": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_size_t]),
    "dlg_hip_host_alloc": (_c.c_int, [_c.c_size_t, _c.POINTER(_c.c_void_p)]),
    "dlg_hip_host_free": (_c.c_int, [_c.c_void_p]),
    "dlg_hip_h2d_async": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_size_t]),
    "dlg_hip_compile": (_c.c_int, [_c.c_char_p, _c.c_char_p, _c.POINTER(_c.c_char_p), _c.c_int,
                                   _c.POINTER(_c.c_void_p), _c.POINTER(_c.c_size_t)]),
    "dlg_hip_code_free": (_c.c_int, [_c.c_void_p]),
    "dlg_hip_compile_log": (_c.c_char_p, []),
    "dlg_hip_module_load": (_c.c_int, [_c.c_char_p, _c.c_size_t, _c.c_char_p,
                                       _c.POINTER(_c.c_uint64)]),
    "dlg_hip_launch": (_c.c_int, [_c.c_uint64] + [_c.c_uint32] * 7 + [_c.c_char_p, _c.c_size_t]),
    "dlg_hip_kernel_attrs": (_c.c_int, [_c.c_uint64] + [_c.POINTER(_c.c_int32)] * 4),
    "dlg_hip_reduce_full": (_c.c_int, [_c.c_uint64, _c.c_uint64, _c.c_void_p, _c.c_uint64, _c.c_uint32, _c.c_float,
                                       _c.c_void_p, _c.c_void_p, _c.c_size_t]),
    "dlg_hip_reduce_full_static": (_c.c_int, [_c.c_uint64, _c.c_uint64, _c.c_void_p, _c.c_uint64, _c.c_uint32, _c.c_float,
                                              _c.c_void_p]),
    "dlg_hip_arena_create": (_c.c_int, [_c.POINTER(_c.c_uint64)]),
    "dlg_hip_arena_set": (_c.c_int, [_c.c_uint64]),
    "dlg_hip_arena_reserve": (_c.c_int, [_c.c_uint64]),
    "dlg_hip_arena_destroy": (_c.c_int, [_c.c_uint64]),
    "dlg_hip_graph_begin": (_c.c_int, []),
    "dlg_hip_graph_end": (_c.c_int, [_c.POINTER(_c.c_uint64), _c.POINTER(_c.c_uint64)]),
    "dlg_hip_graph_launch": (_c.c_int, [_c.c_uint64]),
    "dlg_hip_graph_destroy": (_c.c_int, [_c.c_uint64]),
    "dlg_hip_sync": (_c.c_int, []),
    "dlg_hip_event_create": (_c.c_int, [_c.POINTER(_c.c_uint64)]),
    "dlg_hip_event_record": (_c.c_int, [_c.c_uint64]),
    "dlg_hip_event_sync": (_c.c_int, [_c.c_uint64]),
    "dlg_hip_event_elapsed_ms": (_c.c_int, [_c.c_uint64, _c.c_uint64, _c.POINTER(_c.c_float)]),
    "dlg_hip_event_destroy": (_c.c_int, [_c.c_uint64]),
    "dlg_hip_last_error": (_c.c_char_p, []),
}
EXPORTS = tuple(_SIGS)


class _Props(ctypes.Structure):
    _fields_ = [("name", _c.c_char * 128), ("arch", _c.c_char * 64),
                ("compute_units", _c.c_int32), ("wavefront_size", _c.c_int32),
                ("clock_khz", _c.c_int32), ("mem_clock_khz", _c.c_int32),
                ("mem_bus_bits", _c.c_int32), ("lds_bytes", _c.c_int32),
                ("l2_bytes", _c.c_int32), ("reserved", _c.c_int32),
                ("total_mem", _c.c_uint64)]


class HipError(RuntimeError):
    pass


class HipLib:
    """include/dlgrad_hip.h as methods.  `binding` is "cffi" or "ctypes"."""

    def __init__(self, path: str = LIB_PATH, prefer_cffi: bool = True) -> None:
        if not os.path.exists(path):
            raise HipError(
                f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(the hip device has no CPU fallback)")
        self.path = path
        self.binding = "ctypes"
        self._cffi = None
        if prefer_cffi:
            try:
                import cffi  # noqa: F401  (absent on many ROCm images)
                self._load_cffi(path)
                self.binding = "cffi"
            except ImportError:
                pass
        if self.binding == "ctypes":
            self._lib = ctypes.CDLL(path)
            for name, (res, args) in _SIGS.items():
                fn = getattr(self._lib, name)
                fn.restype, fn.argtypes = res, args
            self._alloc_box = ctypes.c_void_p()
            self._alloc_ref = ctypes.byref(self._alloc_box)
            self.raw_launch = self._lib.dlg_hip_launch      # (handle, gx,gy,gz, bx,by,bz, shmem, args, size)

    # -- cffi binding: same calls, the header text is the cdef ------------------------
    def _load_cffi(self, path: str) -> None:
        import re

        from cffi import FFI
        ffi = FFI()
        text = open(HEADER_PATH).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)          # comments
        text = re.sub(r"^\s*#.*$", "", text, flags=re.M)           # preprocessor lines
        text = text.replace('extern "C" {', "").rstrip().rstrip("}")
        ffi.cdef(text)
        self._cffi = ffi
        self._lib = ffi.dlopen(path)
        self.raw_launch = self._lib.dlg_hip_launch

    # -- helpers -----------------------------------------------------------------------
    def function_address(self, name: str) -> int:
        """Where an exported function lives in this process (for a compiled binding that calls it directly)."""
        if self._cffi is not None:
            return int(self._cffi.cast("uintptr_t", self._cffi.addressof(self._lib, name)))
        return ctypes.cast(getattr(self._lib, name), ctypes.c_void_p).value

    def last_error(self) -> str:
        e = self._lib.dlg_hip_last_error()
        if self._cffi is not None:
            e = self._cffi.string(e)
        return e.decode(errors="replace") if e else ""

    def _check(self, rc: int, exc: type = HipError) -> None:
        if rc != 0:
            raise exc(f"{self.last_error()} [rc={rc}]")

    def _out(self, ctype, cdecl: str):
        """A one-element out-parameter and a reader for it."""
        if self._cffi is not None:
            box = self._cffi.new(cdecl + "[1]")
            return box, (lambda: int(self._cffi.cast("uintptr_t", box[0])) if "*" in cdecl else box[0])
        box = ctype()
        return ctypes.byref(box), (lambda: box.value or 0)

    # -- lifetime ------------------------------------------------------------------------
    def device_count(self) -> int:
        ref, get = self._out(ctypes.c_int, "int")
        rc = self._lib.dlg_hip_device_count(ref)
        return get() if rc == 0 else 0

    def init(self, device: int = 0) -> None:
        self._check(self._lib.dlg_hip_init(device))

    def shutdown(self) -> None:
        self._lib.dlg_hip_shutdown()

    def props(self) -> dict:
        if self._cffi is not None:
            p = self._cffi.new("dlg_hip_props_t *")
            self._check(self._lib.dlg_hip_props(p))
            s = self._cffi.string
            d = {k: getattr(p, k) for k in ("compute_units", "wavefront_size", "clock_khz",
                                            "mem_clock_khz", "mem_bus_bits", "lds_bytes",
                                            "l2_bytes", "total_mem")}
            d["name"], d["arch"] = s(p.name).decode(), s(p.arch).decode()
            return d
        p = _Props()
        self._check(self._lib.dlg_hip_props(ctypes.byref(p)))
        d = {k: getattr(p, k) for k, _ in _Props._fields_ if k != "reserved"}
        d["name"], d["arch"] = p.name.decode(), p.arch.decode()
        return d

    # -- memory --------------------------------------------------------------------------
    def alloc(self, nbytes: int, zero: bool = False) -> int:
        fn = self._lib.dlg_hip_alloc_zero if zero else self._lib.dlg_hip_alloc
        if self._cffi is not None:
            ref, get = self._out(ctypes.c_void_p, "void *")
            rc = fn(nbytes, ref)
            self._check(rc, HipError if rc == -9 else MemoryError)      # -9: refused inside a capture
            return get()
        box = self._alloc_box                     # one reusable out-parameter: this runs per op
        rc = fn(nbytes, self._alloc_ref)
        if rc != 0:
            self._check(rc, HipError if rc == -9 else MemoryError)
        return box.value or 0

    def free(self, ptr: int) -> None:
        self._lib.dlg_hip_free(self._vp(ptr) if self._cffi is not None else ptr)

    def fill_f32(self, ptr: int, value: float, count: int) -> None:
        self._check(self._lib.dlg_hip_fill_f32(self._vp(ptr), value, count))

    def pool_stats(self) -> tuple[int, int, int]:
        outs = [self._out(ctypes.c_uint64, "uint64_t") for _ in range(3)]
        self._lib.dlg_hip_pool_stats(*[o[0] for o in outs])
        return tuple(int(o[1]()) for o in outs)

    def pool_trim(self) -> None:
        self._check(self._lib.dlg_hip_pool_trim())

    def _vp(self, addr: int):
        if self._cffi is not None:
            return self._cffi.cast("void *", addr)
        return ctypes.c_void_p(addr)

    # -- transfers -----------------------------------------------------------------------
    def h2d(self, dst: int, host_addr: int, nbytes: int) -> None:
        self._check(self._lib.dlg_hip_h2d(self._vp(dst), self._vp(host_addr), nbytes))

    def d2h(self, host_addr: int, src: int, nbytes: int) -> None:
        self._check(self._lib.dlg_hip_d2h(self._vp(host_addr), self._vp(src), nbytes))

    def d2d(self, dst: int, src: int, nbytes: int) -> None:
        self._check(self._lib.dlg_hip_d2d(self._vp(dst), self._vp(src), nbytes))

    def host_alloc(self, nbytes: int) -> int:
        ref, get = self._out(ctypes.c_void_p, "void *")
        self._check(self._lib.dlg_hip_host_alloc(nbytes, ref), MemoryError)
        return get() or 0

    def host_free(self, ptr: int) -> None:
        self._check(self._lib.dlg_hip_host_free(self._vp(ptr)))

    def h2d_async(self, dst: int, pinned_addr: int, nbytes: int) -> None:
        self._check(self._lib.dlg_hip_h2d_async(self._vp(dst), self._vp(pinned_addr), nbytes))

    # -- kernels -------------------------------------------------------------------------
    def compile(self, source: str, name: str, options: list[str]) -> bytes:
        """hiprtc: HIP source -> code object bytes.  RuntimeError carries the log."""
        bopts = [o.encode() for o in options]
        if self._cffi is not None:
            ffi = self._cffi
            keep = [ffi.new("char[]", o) for o in bopts]
            arr = ffi.new("char *[]", keep)
            code, size = ffi.new("void *[1]"), ffi.new("size_t[1]")
            rc = self._lib.dlg_hip_compile(source.encode(), name.encode(), arr, len(bopts), code, size)
            if rc != 0:
                log = ffi.string(self._lib.dlg_hip_compile_log()).decode(errors="replace")
                raise RuntimeError(f"Compilation failed:\n{log}\n{self.last_error()}")
            data = bytes(ffi.buffer(code[0], size[0]))
            self._lib.dlg_hip_code_free(code[0])
            return data
        arr = (ctypes.c_char_p * len(bopts))(*bopts)
        code, size = ctypes.c_void_p(), ctypes.c_size_t()
        rc = self._lib.dlg_hip_compile(source.encode(), name.encode(), arr, len(bopts),
                                       ctypes.byref(code), ctypes.byref(size))
        if rc != 0:
            log = (self._lib.dlg_hip_compile_log() or b"").decode(errors="replace")
            raise RuntimeError(f"Compilation failed:\n{log}\n{self.last_error()}")
        data = ctypes.string_at(code, size.value)
        self._lib.dlg_hip_code_free(code)
        return data

    def module_load(self, code: bytes, kernel_name: str) -> int:
        ref, get = self._out(ctypes.c_uint64, "uint64_t")
        self._check(self._lib.dlg_hip_module_load(code, len(code), kernel_name.encode(), ref))
        return int(get())

    def launch(self, handle: int, grid: tuple, block: tuple, args: bytes, shared: int = 0) -> None:
        rc = self._lib.dlg_hip_launch(handle, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                      shared, args, len(args))
        if rc != 0:
            self._check(rc)

    def kernel_attrs(self, handle: int) -> dict:
        outs = [self._out(ctypes.c_int32, "int32_t") for _ in range(4)]
        self._check(self._lib.dlg_hip_kernel_attrs(handle, *[o[0] for o in outs]))
        return dict(zip(("num_regs", "lds_bytes", "scratch_bytes", "max_threads"),
                        (int(o[1]()) for o in outs)))

    def reduce_full(self, k_stage: int, k_fold: int, x: int, n: int, vec: int, divisor: float, out: int,
                    workspace: int, workspace_bytes: int) -> None:
        """Sum or max of n floats at x into out[0] / divisor: both launches in one call."""
        rc = self._lib.dlg_hip_reduce_full(k_stage, k_fold, self._vp(x), n, vec, divisor, self._vp(out),
                                           self._vp(workspace), workspace_bytes)
        if rc != 0:
            self._check(rc)

    def reduce_full_static(self, k_stage: int, k_fold: int, x: int, n: int, vec: int, divisor: float, out: int) -> None:
        """reduce_full with the partial results in the library's static device array: allocates nothing."""
        rc = self._lib.dlg_hip_reduce_full_static(k_stage, k_fold, self._vp(x), n, vec, divisor, self._vp(out))
        if rc != 0:
            self._check(rc)

    # -- arenas and graphs ----------------------------------------------------------------
    def arena_create(self) -> int:
        ref, get = self._out(ctypes.c_uint64, "uint64_t")
        self._check(self._lib.dlg_hip_arena_create(ref))
        return int(get())

    def arena_set(self, arena: int) -> None:
        self._check(self._lib.dlg_hip_arena_set(arena))

    def arena_reserve(self, arena: int) -> None:
        rc = self._lib.dlg_hip_arena_reserve(arena)
        self._check(rc, MemoryError if rc == -3 else HipError)

    def arena_destroy(self, arena: int) -> None:
        self._check(self._lib.dlg_hip_arena_destroy(arena))

    def graph_begin(self) -> None:
        self._check(self._lib.dlg_hip_graph_begin())

    def graph_end(self) -> tuple[int, int]:
        g, gget = self._out(ctypes.c_uint64, "uint64_t")
        n, nget = self._out(ctypes.c_uint64, "uint64_t")
        self._check(self._lib.dlg_hip_graph_end(g, n))
        return int(gget()), int(nget())

    def graph_abandon(self) -> None:
        null = self._cffi.NULL if self._cffi is not None else None
        self._lib.dlg_hip_graph_end(null, null)

    def graph_launch(self, graph: int) -> None:
        self._check(self._lib.dlg_hip_graph_launch(graph))

    def graph_destroy(self, graph: int) -> None:
        self._lib.dlg_hip_graph_destroy(graph)

    # -- ordering and timing ---------------------------------------------------------------
    def sync(self) -> None:
        self._check(self._lib.dlg_hip_sync())

    def event_create(self) -> int:
        ref, get = self._out(ctypes.c_uint64, "uint64_t")
        self._check(self._lib.dlg_hip_event_create(ref))
        return int(get())

    def event_record(self, ev: int) -> None:
        self._check(self._lib.dlg_hip_event_record(ev))

    def event_sync(self, ev: int) -> None:
        self._check(self._lib.dlg_hip_event_sync(ev))

    def event_elapsed_ms(self, start: int, stop: int) -> float:
        ref, get = self._out(ctypes.c_float, "float")
        self._check(self._lib.dlg_hip_event_elapsed_ms(start, stop, ref))
        return float(get())

    def event_destroy(self, ev: int) -> None:
        self._lib.dlg_hip_event_destroy(ev)


_lib: HipLib | None = None


def get_lib() -> HipLib:
    global _lib
    if _lib is None:
        _lib = HipLib()
    return _lib
