"""TEST INFRASTRUCTURE -- numpy-level front end of the C restatement.

Each function does what the matching wrapper in /root/reference/dlgrad/runtime/cpu.py
does around its C call -- output allocation and zero-filling, stride packing, int
truncation of scalar arguments, kernel choice by rank -- with numpy arrays in place
of cffi pointers.  Arrays are fp32 and C-contiguous, as Buffers always are.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from oracle import build as _build

_lib = None
_I = C.POINTER(C.c_int)
_F = C.c_void_p


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(_build.ensure())
    return _lib


def _ia(vals) -> "C.Array":
    vals = [int(v) for v in vals]
    return (C.c_int * max(len(vals), 1))(*vals)


def _p(a: np.ndarray):
    return C.c_void_p(a.ctypes.data)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def strides_of(shape) -> tuple:
    out, acc = [], 1
    for d in reversed(tuple(shape)):
        out.append(acc)
        acc *= d
    return tuple(reversed(out))


def bcast_shape(s1, s2) -> tuple:
    return tuple(np.broadcast_shapes(tuple(s1), tuple(s2)))


def bcast_strides(out_shape, in_shape) -> tuple:
    """Effective strides with 0 on stretched dims (helpers.py:276-309)."""
    pad = len(out_shape) - len(in_shape)
    shape = (1,) * pad + tuple(in_shape)
    st = (0,) * pad + strides_of(in_shape)
    return tuple(0 if (i == 1 and o > 1) else s for o, i, s in zip(out_shape, shape, st))


# ---- cpu.py:257-311, :784-791, :906-908 --------------------------------------------------
def binary(op: str, x, y) -> np.ndarray:
    x, y = _f32(x), _f32(y)
    out_shape = bcast_shape(x.shape, y.shape)
    out = np.empty(out_shape, np.float32)
    fn = getattr(lib(), f"ref_{op}")
    fn(_p(x), _p(y), _p(out), len(out_shape), _ia(out_shape), _ia(bcast_strides(out_shape, x.shape)),
       _ia(bcast_strides(out_shape, y.shape)))
    return out


# ---- cpu.py:834-862 ----------------------------------------------------------------------------
def cmp_le(x, y, out_shape) -> np.ndarray:
    x, y = _f32(x), _f32(y)
    out = np.empty(out_shape, np.float32)
    xs = [0 if d == 1 else 1 for d in x.shape]
    ys = [0 if d == 1 else 1 for d in y.shape]
    lib().ref_cmp_le(_p(x), _p(y), _p(out), _ia(out_shape), _ia(xs), _ia(ys), _ia(strides_of(out_shape)))
    return out


# ---- cpu.py:313-331, :370-428, :464-502 -----------------------------------------------------------
def unary(op: str, x, val=None) -> np.ndarray:
    x = _f32(x)
    out = np.empty_like(x)
    fn = getattr(lib(), f"ref_{op}")
    if op == "pow":
        fn(_p(x), _p(out), x.size, int(val))       # cpu.py:500: int(val)
    else:
        fn(_p(x), _p(out), x.size)
    return out


def clamp(x, min_val=None, max_val=None) -> np.ndarray:
    x = _f32(x)
    out = np.empty_like(x)
    lib().ref_clamp(_p(x), _p(out), x.size, int(min_val is not None),
                    C.c_float(0.0 if min_val is None else float(min_val)), int(max_val is not None),
                    C.c_float(0.0 if max_val is None else float(max_val)))
    return out


# ---- cpu.py:604-761 ---------------------------------------------------------------------------------
def reduce(op: str, x, dim: int = -1) -> np.ndarray:
    """dim == -1 (or None): all elements -> 0-d.  Otherwise that axis is removed."""
    x = _f32(x)
    if dim is None or dim == -1:
        out = np.empty((), np.float32)
        getattr(lib(), f"ref_reduce_{op}")(_p(x), _p(out), x.size)
        return out
    if dim < 0:
        dim += x.ndim
    out_shape = tuple(d for i, d in enumerate(x.shape) if i != dim)
    out = np.empty(out_shape, np.float32)
    getattr(lib(), f"ref_reduce_{op}_axis")(_p(x), _p(out), x.ndim, dim, _ia(x.shape),
                                            _ia(strides_of(x.shape)), _ia(strides_of(out_shape)))
    return out


# ---- cpu.py:910-959 -------------------------------------------------------------------------------------
def argmax(x, dim) -> np.ndarray:
    x = _f32(x)
    if dim is None:
        shape, st, ndim, dim, out_shape = (x.size,), (1,), 1, 0, (1,)
    else:
        if dim < 0:
            dim += x.ndim
        shape, st, ndim = x.shape, strides_of(x.shape), x.ndim
        out_shape = tuple(d for i, d in enumerate(x.shape) if i != dim)
    out = np.empty(out_shape, np.float32)
    lib().ref_argmax_axis(_p(x), _p(out), ndim, dim, _ia(shape), _ia(st), _ia(strides_of(out_shape)))
    return out


# ---- cpu.py:333-368 -----------------------------------------------------------------------------------------
def permute(x, order) -> np.ndarray:
    x = _f32(x)
    out_shape = tuple(x.shape[i] for i in order)
    st = strides_of(x.shape)
    out = np.empty(out_shape, np.float32)
    lib().ref_permute(_p(x), _p(out), x.ndim, _ia(out_shape), _ia([st[i] for i in order]),
                      _ia(strides_of(out_shape)))
    return out


# ---- cpu.py:864-903, :793-831 -----------------------------------------------------------------------------------
def where(cond, x, y) -> np.ndarray:
    cond, x, y = _f32(cond), _f32(x), _f32(y)
    out_shape = bcast_shape(bcast_shape(x.shape, y.shape), cond.shape)
    out = np.empty(out_shape, np.float32)
    lib().ref_where(_p(cond), _p(x), _p(y), _p(out), len(out_shape), _ia(out_shape),
                    _ia(bcast_strides(out_shape, cond.shape)), _ia(bcast_strides(out_shape, x.shape)),
                    _ia(bcast_strides(out_shape, y.shape)), _ia(strides_of(out_shape)))
    return out


def masked_fill(x, mask, val: float) -> np.ndarray:
    x, mask = _f32(x), _f32(mask)
    out_shape = bcast_shape(x.shape, mask.shape)
    out = np.empty(out_shape, np.float32)
    lib().ref_masked_fill(_p(x), _p(mask), _p(out), len(out_shape), _ia(out_shape),
                          _ia(bcast_strides(out_shape, x.shape)), _ia(bcast_strides(out_shape, mask.shape)),
                          _ia(strides_of(out_shape)), C.c_float(val))
    return out


# ---- cpu.py:504-602 ---------------------------------------------------------------------------------------------
def matmul(x, y) -> np.ndarray:
    """x, y already padded to equal rank 2, 3 or 4 (buffer.py:231-235)."""
    x, y = _f32(x), _f32(y)
    assert x.ndim == y.ndim and x.ndim in (2, 3, 4)
    if x.ndim == 2:
        out = np.zeros((x.shape[0], y.shape[1]), np.float32)          # init_with_scalar(0)
        lib().ref_matmul_2d(_p(x), _p(y), _p(out), _ia(x.shape), _ia(strides_of(x.shape)),
                            _ia(y.shape), _ia(strides_of(y.shape)))
        return out
    if x.ndim == 3:
        B = max(x.shape[0], y.shape[0])
        M, K, N = x.shape[1], x.shape[2], y.shape[2]
        out = np.zeros((B, M, N), np.float32)                          # calloc
        sx, sy = list(strides_of(x.shape)), list(strides_of(y.shape))
        if x.shape[0] == 1 and B > 1:
            sx[0] = 0
        if y.shape[0] == 1 and B > 1:
            sy[0] = 0
        lib().ref_matmul_3d(_p(x), _p(y), _p(out), B, M, K, N, _ia(sx), _ia(sy), _ia(strides_of(out.shape)))
        return out
    B, Cc = max(x.shape[0], y.shape[0]), max(x.shape[1], y.shape[1])
    M, K, N = x.shape[2], x.shape[3], y.shape[3]
    out = np.zeros((B, Cc, M, N), np.float32)
    sx, sy = list(strides_of(x.shape)), list(strides_of(y.shape))
    for d, big in ((0, B), (1, Cc)):
        if x.shape[d] == 1 and big > 1:
            sx[d] = 0
        if y.shape[d] == 1 and big > 1:
            sy[d] = 0
    lib().ref_matmul_4d(_p(x), _p(y), _p(out), _ia([B, Cc, M, K, N]), _ia(sx), _ia(sy),
                        _ia(strides_of(out.shape)))
    return out


# ---- cpu.py:1027-1061 ----------------------------------------------------------------------------------------------
def embedding(table, idx) -> np.ndarray:
    table, idx = _f32(table), _f32(idx)
    W = table.shape[-1]
    out = np.empty(idx.shape + (W,), np.float32)
    lib().ref_embedding(_p(table), _p(idx), _p(out), idx.size, W)
    return out


def embedding_backward(table_shape, idx, upstream, float_index: bool = False) -> np.ndarray:
    """float_index=True is the reference's literal expression (index formed in fp32,
    wrong above 2**24); the default forms it in integers."""
    idx, upstream = _f32(idx), _f32(upstream)
    out = np.zeros(table_shape, np.float32)                            # init_with_scalar(0)
    fn = lib().ref_embedding_backward if float_index else lib().ref_embedding_backward_int
    fn(_p(out), _p(upstream), _p(idx), idx.size, table_shape[-1])
    return out


# ---- cpu.py:961-1000 ---------------------------------------------------------------------------------------------------
def ce_forward(x, target) -> np.ndarray:
    x, target = _f32(x), _f32(target)
    out = np.empty((x.shape[0],), np.float32)
    lib().ref_ce_forward(_p(x), _p(target), _p(out), x.shape[0], _ia(strides_of(x.shape)))
    return out


def ce_backward_(x: np.ndarray, target) -> None:
    """In place on `x` (must be a C-contiguous fp32 array)."""
    assert x.dtype == np.float32 and x.flags.c_contiguous
    target = _f32(target)
    lib().ref_ce_backward(_p(x), _p(target), _ia(x.shape), _ia(strides_of(x.shape)))


# ---- cpu.py:216-254 -----------------------------------------------------------------------------------------------------
def arange(shape) -> np.ndarray:
    out = np.empty(shape, np.float32)
    lib().ref_arange(_p(out), out.size)
    return out


def full(shape, fill_value, strict: bool = True) -> np.ndarray:
    out = np.empty(shape, np.float32)
    if strict:
        lib().ref_full(_p(out), out.size, int(fill_value))             # cpu.py:252: int(fill_value)
    else:
        lib().ref_full_f(_p(out), out.size, C.c_float(fill_value))
    return out


def uniform(shape, low: float, high: float, seed: int, seq: int = 54) -> np.ndarray:
    out = np.empty(shape, np.float32)
    lib().ref_uniform(_p(out), out.size, C.c_float(low), C.c_float(high), C.c_uint64(seed), C.c_uint64(seq))
    return out


def pcg32_raw(n: int, seed: int, seq: int) -> np.ndarray:
    out = np.empty(n, np.uint32)
    lib().ref_pcg32_raw(_p(out), n, C.c_uint64(seed), C.c_uint64(seq))
    return out
