"""TEST INFRASTRUCTURE -- a `cpu` runtime for the dispatch table, backed by the C restatement.

Registers one entry per (op, Device.CPU) pair, the way /root/reference/dlgrad/runtime/cpu.py
does, so that whole graphs (the MLP step, the GPT step) can run on the reference's CPU
kernels and be compared with the hip device.  Pointers are `HostPtr` (a flat fp32 numpy
array); everything numeric happens in oracle/cref.py.
"""
from __future__ import annotations

import numpy as np

from dlgrad_amd.buffer import Buffer
from dlgrad_amd.device import Device
from dlgrad_amd.dispatch import dispatcher
from dlgrad_amd.helpers import STRICT_REFERENCE, BinaryOps, BufferOps, CustomOps, UnaryOps
from oracle import cref


class HostPtr:
    __slots__ = ("arr",)

    def __init__(self, arr: np.ndarray) -> None:
        self.arr = np.ascontiguousarray(arr, dtype=np.float32).reshape(-1)

    def __add__(self, n: int) -> "HostPtr":
        v = HostPtr.__new__(HostPtr)
        v.arr = self.arr[int(n):]
        return v


def _np(b: Buffer) -> np.ndarray:
    if b.is_host_scalar:
        return np.array(b.ptr.value, dtype=np.float32)
    return b.ptr.arr[:b.numel].reshape(b.shape)


def _reg(op):
    return dispatcher.register(op, Device.CPU)


class CPU:
    _seed = int.from_bytes(__import__("os").urandom(8), "little")
    _stream = 0

    @staticmethod
    def manual_seed(seed: int) -> None:
        """Same convention as the hip runtime: call k after this draws PCG32 stream k of `seed`."""
        CPU._seed, CPU._stream = int(seed) & ((1 << 64) - 1), 0

    @staticmethod
    @_reg(BufferOps.CREATE)
    def create(data: np.ndarray, into: Buffer | None = None) -> HostPtr:
        if into is not None:
            into.ptr.arr[:data.size] = np.asarray(data, dtype=np.float32).reshape(-1)
            return into.ptr
        return HostPtr(np.array(data, dtype=np.float32, copy=True))

    @staticmethod
    @_reg(CustomOps.FROM_U8)
    def from_u8(data: np.ndarray) -> HostPtr:
        return HostPtr(np.asarray(data, dtype=np.uint8).astype(np.float32))

    @staticmethod
    @_reg(CustomOps.ROW_STORE)
    def row_store(dst: Buffer, src: Buffer, idx: Buffer, rows: int, width: int) -> None:
        i = float(idx.ptr.arr[0])
        if 0 <= i < rows:
            dst.ptr.arr[int(i) * width:(int(i) + 1) * width] = src.ptr.arr[:width]

    @staticmethod
    @_reg(CustomOps.COPY_INTO)
    def copy_into(dst: Buffer, src: Buffer) -> None:
        dst.ptr.arr[:dst.numel] = src.ptr.arr[:src.numel]

    @staticmethod
    @_reg(CustomOps.TO_HOST)
    def to_host(x: Buffer) -> np.ndarray:
        return _np(x).copy()

    @staticmethod
    @_reg(CustomOps.PRINT)
    def show(x: Buffer) -> None:
        print(_np(x))

    @staticmethod
    @_reg(BufferOps.UNIFORM)
    def uniform(shape: tuple, low: float = 0.0, high: float = 1.0) -> HostPtr:
        seq, CPU._stream = CPU._stream, CPU._stream + 1
        return HostPtr(cref.uniform(shape, low, high, seed=CPU._seed, seq=seq))

    @staticmethod
    @_reg(BufferOps.FULL)
    def full(shape: tuple, fill_value: float) -> HostPtr:
        return HostPtr(cref.full(shape, fill_value, strict=STRICT_REFERENCE))

    @staticmethod
    @_reg(BufferOps.ARANGE)
    def arange(shape: tuple) -> HostPtr:
        return HostPtr(cref.arange(shape))

    @staticmethod
    @_reg(BinaryOps.CMP)
    def cmp(x: Buffer, y: Buffer, out_shape: tuple, mode: str) -> HostPtr:
        assert mode == "<="
        return HostPtr(cref.cmp_le(_np(x), _np(y), out_shape))

    @staticmethod
    @_reg(UnaryOps.POW)
    def pow(x: Buffer, val: float) -> HostPtr:
        return HostPtr(cref.unary("pow", _np(x), val))

    @staticmethod
    @_reg(UnaryOps.CLAMP)
    def clamp(x: Buffer, min_val, max_val) -> HostPtr:
        return HostPtr(cref.clamp(_np(x), min_val, max_val))

    @staticmethod
    @_reg(UnaryOps.ARGMAX)
    def argmax(x: Buffer, dim: int) -> HostPtr:
        return HostPtr(cref.argmax(_np(x), dim))

    @staticmethod
    @_reg(UnaryOps.PERMUTE)
    def permute(x: Buffer, order: tuple) -> HostPtr:
        return HostPtr(cref.permute(_np(x), order))

    @staticmethod
    @_reg(UnaryOps.WHERE)
    def where(cond: Buffer, x: Buffer, y: Buffer) -> HostPtr:
        return HostPtr(cref.where(_np(cond), _np(x), _np(y)))

    @staticmethod
    @_reg(UnaryOps.MASKED_FILL)
    def masked_fill(x: Buffer, mask: Buffer, val: float, out_shape: tuple) -> HostPtr:
        return HostPtr(cref.masked_fill(_np(x), _np(mask), val))

    @staticmethod
    @_reg(BinaryOps.MATMUL)
    def matmul(x: Buffer, y: Buffer) -> HostPtr:
        return HostPtr(cref.matmul(_np(x), _np(y)))

    @staticmethod
    @_reg(CustomOps.EMBEDDING)
    def embedding(x: Buffer, idx: Buffer, out_numel: int, backward: bool = False,
                  upstream_grad: Buffer = None) -> HostPtr:
        if backward:
            return HostPtr(cref.embedding_backward(x.shape, _np(idx), _np(upstream_grad)))
        return HostPtr(cref.embedding(_np(x), _np(idx)))

    @staticmethod
    @_reg(CustomOps.CE_FORWARD)
    def ce_forward(x: Buffer, y: Buffer) -> HostPtr:
        return HostPtr(cref.ce_forward(_np(x), _np(y)))

    @staticmethod
    @_reg(CustomOps.CE_BACKWARD)
    def ce_backward(x: Buffer, target: Buffer) -> None:
        cref.ce_backward_(_np(x), _np(target))          # a view of x's own memory: in place


def _register_tables() -> None:
    for op, name in ((BinaryOps.ADD, "add"), (BinaryOps.SUB, "sub"), (BinaryOps.MUL, "mul"),
                     (BinaryOps.DIV, "div"), (BinaryOps.GT, "gt"), (BinaryOps.GTE, "gte"),
                     (BinaryOps.EQT, "eq")):
        dispatcher.register(op, Device.CPU)(
            lambda x, y, _n=name: HostPtr(cref.binary(_n, _np(x), _np(y))))
    for op, name in ((UnaryOps.NEG, "neg"), (UnaryOps.EXP, "exp"), (UnaryOps.LOG, "log"),
                     (UnaryOps.SQRT, "sqrt"), (UnaryOps.RSQRT, "rsqrt"), (UnaryOps.RELU, "relu")):
        dispatcher.register(op, Device.CPU)(lambda x, _n=name: HostPtr(cref.unary(_n, _np(x))))
    for op, name in ((UnaryOps.SUM, "sum"), (UnaryOps.MEAN, "mean"), (UnaryOps.MAX, "max")):
        dispatcher.register(op, Device.CPU)(
            lambda x, dim, out=None, _n=name: HostPtr(cref.reduce(_n, _np(x), dim)))


_register_tables()
