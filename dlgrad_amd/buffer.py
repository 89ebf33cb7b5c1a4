"""Buffer: a pointer plus shape metadata, and the place where ops pick a runtime.

Same role and method names as dlgrad/buffer.py:35-565, with one deliberate
difference that is part of the device boundary: the reference hard-wires many
ops to Device.CPU (creation ops, masked_fill, mean, permute, rsqrt, clamp,
where, argmax, comparisons, cross-entropy and embedding helpers; buffer.py:48,
:104-130, :204, :292-297, :322-328, :367-400, :454-528), which only works where
host and device share memory.  Here *every* op goes to `self.device`, so a
Buffer that lives in HBM never needs a host round trip.

`ptr` is opaque to this file: the runtime that made it knows what it is (a
`DevicePtr` for HIP).  Python floats that enter an expression become 0-d
Buffers whose `ptr` is a `HostScalar`; runtimes receive those by value instead
of uploading four bytes (the reference keeps them in a host `float[1]`,
buffer.py:86-90).  Buffers are always contiguous: `stride` is derived from
`shape`, and permutations materialise, exactly as in the reference.
"""
from __future__ import annotations

from functools import lru_cache

import numpy as np

from dlgrad_amd.device import Device, as_device
from dlgrad_amd.dispatch import dispatcher
from dlgrad_amd.dtype import CDataPtr, DType, Scalar
from dlgrad_amd.helpers import (
    BinaryOps,
    BufferOps,
    CustomOps,
    UnaryOps,
    broadcast_shapes,
    cal_sum_max_out_shape,
    calculate_stride,
    check_broadcast,
    get_broadcast_shape,
    prod_,
)


_new_buffer = object.__new__
_dispatch_table = dispatcher._dispatch_table      # (op, device) -> runtime function: the table dispatcher.dispatch reads


class HostScalar:
    """One fp32 value that lives on the host and is passed to kernels by value."""
    __slots__ = ("value",)

    def __init__(self, value: float) -> None:
        self.value = np.float32(value)

    def __float__(self) -> float:
        return float(self.value)

    def __repr__(self) -> str:
        return f"HostScalar({float(self.value)!r})"


@lru_cache(maxsize=16384)
def _shape_info(shape: tuple) -> tuple:
    """(numel, stride, ndim, nbytes) of a contiguous fp32 array of this shape."""
    n = prod_(shape)
    return n, calculate_stride(shape), len(shape), n * 4


def _is_scalar(v) -> bool:
    c = v.__class__
    return c is float or c is int or (c is not bool and isinstance(v, (int, float, np.floating)) and not isinstance(v, bool))


# 0-d host values never reach a device: scalar-with-scalar arithmetic is done here in
# fp32 (the reference runs its zero-loop C kernels on them, cpu_kernel.py:47-48).
_f32 = np.float32
_HOST_BINARY = {
    BinaryOps.ADD: lambda a, b: a + b, BinaryOps.SUB: lambda a, b: a - b,
    BinaryOps.MUL: lambda a, b: a * b, BinaryOps.DIV: lambda a, b: a / b,
    BinaryOps.GT: lambda a, b: _f32(a > b), BinaryOps.GTE: lambda a, b: _f32(a >= b),
    BinaryOps.EQT: lambda a, b: _f32(a == b),
}
_HOST_UNARY = {
    UnaryOps.NEG: lambda v: -v,
    UnaryOps.EXP: lambda v: _f32(np.exp(np.float64(v))),
    UnaryOps.LOG: lambda v: _f32(np.log(np.float64(v))),
    UnaryOps.SQRT: lambda v: np.sqrt(v),
    UnaryOps.RSQRT: lambda v: _f32(1.0) / np.sqrt(v),
    UnaryOps.POW: lambda v, val: _f32(np.float64(v) ** int(val)),
    UnaryOps.CLAMP: lambda v, min_val, max_val: _f32(
        min(max(v, v if min_val is None else _f32(min_val)), v if max_val is None else _f32(max_val))),
}


_frozen: dict = {}      # id(ptr) -> ptr of allocations that the in-place methods refuse to write (Buffer.freeze)


class Buffer:
    """shape / numel / stride / ndim / dtype / device / nbytes are attributes of the Buffer itself;
    `metadata` (the reference keeps them in a separate BufferMetadata object, buffer.py:24-32, and
    reads and writes them as `buf.metadata.shape`) is the Buffer again, so both spellings work and
    creating a Buffer -- which happens for every op output -- allocates one object, not two."""
    __slots__ = ("ptr", "shape", "numel", "stride", "ndim", "dtype", "device", "nbytes", "__weakref__")

    def __init__(self, data: CDataPtr, shape: tuple, device: str | Device | None = Device.CPU,
                 dtype: str | DType | None = None, **kwargs) -> None:
        self.ptr = data
        shape = tuple(shape)
        if dtype is None or dtype.__class__ is str:
            dtype = DType.from_str(dtype) if dtype else DType.FLOAT32
        if device.__class__ is not Device:
            device = as_device(device)
        n, stride, ndim, nbytes = _shape_info(shape)
        room = getattr(data, "nbytes", None)               # device pointers know how much of their block is left
        if room is not None and nbytes > room:
            raise ValueError(f"a Buffer of shape {shape} needs {nbytes} bytes, the pointer has {room}")
        if kwargs:
            stride, ndim = kwargs.get("stride", stride), kwargs.get("ndim", ndim)
        self.shape, self.numel, self.stride, self.ndim = shape, n, stride, ndim
        self.dtype, self.device, self.nbytes = dtype, device, nbytes

    @property
    def metadata(self) -> "Buffer":
        return self

    @staticmethod
    def fresh(ptr: CDataPtr, shape: tuple, device: Device, dtype: DType = DType.FLOAT32) -> "Buffer":
        """A Buffer around a pointer the runtime has just made for exactly this (tuple) shape: no
        conversions and no size check."""
        b = _new_buffer(Buffer)
        b.ptr, b.shape, b.dtype, b.device = ptr, shape, dtype, device
        b.numel, b.stride, b.ndim, b.nbytes = _shape_info(shape)
        return b

    # ---- plumbing -------------------------------------------------------------------
    def _dispatch(self, op, **kw):
        return _dispatch_table[(op, self.device)](**kw)            # what dispatcher.dispatch does, one call less

    def _like(self, ptr, shape: tuple | None = None, **kw) -> "Buffer":
        if kw or (shape is not None and shape.__class__ is not tuple):
            return Buffer(data=ptr, shape=self.shape if shape is None else shape,
                          device=self.device, dtype=self.dtype, **kw)
        b = _new_buffer(Buffer)
        b.ptr, b.dtype, b.device = ptr, self.dtype, self.device
        if shape is None:
            b.shape, b.numel, b.stride, b.ndim, b.nbytes = self.shape, self.numel, self.stride, self.ndim, self.nbytes
        else:
            b.shape = shape
            b.numel, b.stride, b.ndim, b.nbytes = _shape_info(shape)
            room = getattr(ptr, "nbytes", None)
            if room is not None and b.nbytes > room:
                raise ValueError(f"a Buffer of shape {shape} needs {b.nbytes} bytes, the pointer has {room}")
        return b

    @property
    def is_host_scalar(self) -> bool:
        return self.ptr.__class__ is HostScalar

    def _set_shape(self, shape: tuple) -> None:
        self.shape = tuple(shape)
        self.numel, self.stride, self.ndim, _ = _shape_info(self.shape)

    # ---- host boundary ----------------------------------------------------------------
    @staticmethod
    def from_numpy(arr: np.ndarray, device: Device) -> "Buffer":
        """H2D upload (the reference aliases the numpy memory, tensor.py:112-115)."""
        device = as_device(device)
        return Buffer(data=dispatcher.dispatch(op=BufferOps.CREATE, device=device, data=arr),
                      shape=arr.shape, device=device, dtype=DType.FLOAT32, ndim=arr.ndim)

    @staticmethod
    def from_u8(arr: np.ndarray, device: Device) -> "Buffer":
        """fp32 Buffer holding (float)arr[i] for a uint8 host array: the bytes are uploaded as
        they are and widened where the Buffer lives."""
        device = as_device(device)
        if arr.dtype != np.uint8:
            raise TypeError(f"from_u8 takes uint8 data, got {arr.dtype}")
        return Buffer(data=dispatcher.dispatch(op=CustomOps.FROM_U8, device=device, data=arr),
                      shape=arr.shape, device=device, dtype=DType.FLOAT32, ndim=arr.ndim)

    def numpy(self) -> np.ndarray:
        """D2H copy with this Buffer's shape (buffer.py:67-84 returns a host view)."""
        if self.is_host_scalar:
            return np.array(self.ptr.value, dtype=np.float32).reshape(self.shape)
        return self._dispatch(CustomOps.TO_HOST, x=self)

    def show(self) -> None:
        self._dispatch(CustomOps.PRINT, x=self)

    @staticmethod
    def from_scalar(val: Scalar) -> "Buffer":
        return Buffer.fresh(HostScalar(val), (), Device.CPU)

    # ---- creation -----------------------------------------------------------------------
    @staticmethod
    def uniform(shape: tuple, device: Device, dtype: DType | str, **kwargs) -> "Buffer":
        dtype = DType.from_str(dtype) if isinstance(dtype, str) else dtype
        device = as_device(device)
        if dtype is not DType.FLOAT32:
            raise NotImplementedError("dlgrad only supports float32")
        if not isinstance(shape, tuple):
            raise ValueError("Shape must be a tuple")
        return Buffer(data=dispatcher.dispatch(op=BufferOps.UNIFORM, device=device, shape=shape, **kwargs),
                      shape=shape, device=device, dtype=dtype)

    @staticmethod
    def full(shape: tuple, fill_value: Scalar, device: Device, dtype: DType = DType.FLOAT32) -> "Buffer":
        device = as_device(device)
        return Buffer(data=dispatcher.dispatch(op=BufferOps.FULL, device=device, shape=shape,
                                               fill_value=fill_value),
                      shape=shape, device=device, dtype=dtype)

    @staticmethod
    def arange(shape: tuple, device: Device, dtype: DType = DType.FLOAT32) -> "Buffer":
        device = as_device(device)
        return Buffer(data=dispatcher.dispatch(op=BufferOps.ARANGE, device=device, shape=shape),
                      shape=shape, device=device, dtype=dtype)

    # ---- views (metadata only) --------------------------------------------------------------
    def reshape(self, new_shape: tuple) -> "Buffer":
        new_shape = tuple(new_shape)
        if -1 in new_shape:
            known = -prod_(new_shape)
            new_shape = tuple(self.numel // known if d == -1 else d for d in new_shape)
        if prod_(new_shape) != self.numel:
            raise ValueError(f"Cannot reshape {self.shape} ({self.numel} elements) to {new_shape} "
                             f"({prod_(new_shape)} elements)")
        return self._like(self.ptr, new_shape)

    def unsqueeze(self, dim: list[int] | int) -> None:
        """In place, like the reference (buffer.py:134-151); dim == -1 means 0."""
        if dim == -1:
            dim = 0
        dims = [dim] if isinstance(dim, int) else list(dim)
        if len(set(dims)) != len(dims):
            raise AssertionError(f"duplicate dims not allowed in unsqueeze: {dim}")
        shape = list(self.shape)
        for d in dims:
            assert d <= len(shape), f"Cannot unsqueeze {dim} from {self.shape}"
        for d in sorted(dims, reverse=True):
            shape.insert(d, 1)
        self._set_shape(tuple(shape))

    def squeeze(self, dim: list[int] | int) -> None:
        """In place; dims that are not of extent 1 are left alone (buffer.py:153-165)."""
        for d in ([dim] if isinstance(dim, int) else dim):
            if self.shape[d] == 1:
                shape = list(self.shape)
                del shape[d]
                self._set_shape(tuple(shape))

    # ---- reductions -------------------------------------------------------------------------
    def _reduce(self, op: UnaryOps, dim: int, keepdim: bool) -> "Buffer":
        out_shape = cal_sum_max_out_shape(ndim=self.ndim, dim=dim, inp_shape=self.shape, keepdim=keepdim)
        if dim == -1 and keepdim:
            # helpers.py:205-206 reports the *input* shape here although one element is
            # produced; a shape of ones is what that element can back.
            out_shape = (1,) * self.ndim
        ndim = self.ndim if keepdim else (0 if dim == -1 else self.ndim - 1)
        return self._like(self._dispatch(op, x=self, dim=dim), out_shape, ndim=ndim)

    def sum(self, dim: int = -1, keepdim: bool = False) -> "Buffer":
        return self._reduce(UnaryOps.SUM, dim, keepdim)

    def mean(self, dim: int = -1, keepdim: bool = False) -> "Buffer":
        return self._reduce(UnaryOps.MEAN, dim, keepdim)

    def max(self, dim: int = -1, out: "Buffer" = None, keepdim: bool = False) -> "Buffer":
        return self._reduce(UnaryOps.MAX, dim, keepdim)

    def argmax(self, dim: int) -> "Buffer":
        assert self.ndim == 2, "currently dlgrad supports argmax for 2d only"
        shape = {0: (1, self.shape[1]), 1: (self.shape[0], 1)}.get(dim, (1, 1))
        return self._like(self._dispatch(UnaryOps.ARGMAX, x=self, dim=dim), shape)

    # ---- matmul / layout ----------------------------------------------------------------------
    def _tri(self, tri: str) -> dict:
        """A triangular-structure hint for the product kernels (see HIP.matmul); runtimes that
        do not know it compute the whole product, which gives the same kept values."""
        return {"tri": tri} if tri and self.device is Device.HIP else {}

    def matmul(self, other: "Buffer", tri: str = "", epi: str = "", e: "Buffer | None" = None) -> "Buffer":
        """epi / e (hip only): an element-wise step fused into the store of the result, see HIP.matmul."""
        p1, p2, out_shape = broadcast_shapes(self.shape, other.shape)
        x = self if self.shape == p1 else self._like(self.ptr, p1)
        y = other if other.shape == p2 else other._like(other.ptr, p2)
        kw = {"epi": epi, "e": e} if epi else {}
        return self._like(self._dispatch(BinaryOps.MATMUL, x=x, y=y, **self._tri(tri), **kw), out_shape)

    def matmul_nt(self, other: "Buffer", tri: str = "", epi: str = "", e: "Buffer | None" = None,
                  norm: tuple | None = None) -> "Buffer":
        """self (.., M, K) @ other(.., N, K)^T without materialising the transpose.  norm (hip only, a single
        row): (gain, eps) of an RMS normalisation applied to self on its way into the product, see HIP.matmul."""
        swapped = other.shape[:-2] + (other.shape[-1], other.shape[-2])
        p1, p2, out_shape = broadcast_shapes(self.shape, swapped)
        p2 = p2[:-2] + (p2[-1], p2[-2])
        x = self if self.shape == p1 else self._like(self.ptr, p1)
        y = other if other.shape == p2 else other._like(other.ptr, p2)
        kw = {"epi": epi, "e": e} if epi else {}
        if norm is not None:
            kw["norm"] = norm
            if len(norm) > 2 and norm[2]:                 # also the normalised rows and their 1 / rms
                out, yn, rinv = self._dispatch(CustomOps.MATMUL_NT, x=x, y=y, **self._tri(tri), **kw)
                return self._like(out, out_shape), self._like(yn), self._like(rinv, (self.numel // max(self.shape[-1], 1),))
        return self._like(self._dispatch(CustomOps.MATMUL_NT, x=x, y=y, **self._tri(tri), **kw), out_shape)

    def matmul_tn(self, other: "Buffer", tri: str = "") -> "Buffer":
        """self(.., K, M)^T @ other (.., K, N) without materialising the transpose."""
        swapped = self.shape[:-2] + (self.shape[-1], self.shape[-2])
        p1, p2, out_shape = broadcast_shapes(swapped, other.shape)
        p1 = p1[:-2] + (p1[-1], p1[-2])
        x = self if self.shape == p1 else self._like(self.ptr, p1)
        y = other if other.shape == p2 else other._like(other.ptr, p2)
        return self._like(self._dispatch(CustomOps.MATMUL_TN, x=x, y=y, **self._tri(tri)), out_shape)

    @staticmethod
    def _product_operands(kind: str, a: "Buffer", b: "Buffer") -> tuple:
        """(x, y, ta, tb, out_shape) of a @ b ("nn"), a @ b^T ("nt") or a^T @ b ("tn") with the operands padded
        to one rank, as matmul / matmul_nt / matmul_tn hand them to the runtime."""
        sa = a.shape[:-2] + (a.shape[-1], a.shape[-2]) if kind == "tn" else a.shape
        sb = b.shape[:-2] + (b.shape[-1], b.shape[-2]) if kind == "nt" else b.shape
        p1, p2, out_shape = broadcast_shapes(sa, sb)
        if kind == "tn":
            p1 = p1[:-2] + (p1[-1], p1[-2])
        if kind == "nt":
            p2 = p2[:-2] + (p2[-1], p2[-2])
        x = a if a.shape == p1 else a._like(a.ptr, p1)
        y = b if b.shape == p2 else b._like(b.ptr, p2)
        return x, y, kind == "tn", kind == "nt", out_shape

    @staticmethod
    def matmul_pair(first: tuple, second: tuple) -> tuple["Buffer", "Buffer"]:
        """Two independent products as one launch on the hip device: each is (kind, a, b) or (kind, a, b,
        epi, e) with kind "nn" (a @ b), "nt" (a @ b^T) or "tn" (a^T @ b) and the epilogues of matmul.
        The results are those of the separate calls, bit for bit."""
        specs, shapes = [], []
        for kind, a, b, *rest in (first, second):
            x, y, ta, tb, out_shape = Buffer._product_operands(kind, a, b)
            epi, e = (rest + ["", None])[:2] if rest else ("", None)
            specs.append((x, y, ta, tb, epi, e))
            shapes.append(out_shape)
        a0 = first[1]
        p0, p1 = a0._dispatch(CustomOps.MATMUL_PAIR, first=specs[0], second=specs[1])
        return a0._like(p0, shapes[0]), a0._like(p1, shapes[1])

    def permute(self, order: tuple) -> "Buffer":
        order = tuple(order)
        return self._like(self._dispatch(UnaryOps.PERMUTE, x=self, order=order),
                          tuple(self.shape[i] for i in order))

    def transpose(self, dim0: int, dim1: int) -> "Buffer":
        order = list(range(self.ndim))
        order[dim0], order[dim1] = order[dim1], order[dim0]
        return self.permute(tuple(order))

    # ---- unary --------------------------------------------------------------------------------
    def _unary(self, op: UnaryOps, **kw) -> "Buffer":
        if self.is_host_scalar and op in _HOST_UNARY:
            with np.errstate(all="ignore"):
                return self._like(HostScalar(_HOST_UNARY[op](self.ptr.value, **kw)))
        return self._like(self._dispatch(op, x=self, **kw))

    def exp(self) -> "Buffer":
        return self._unary(UnaryOps.EXP)

    def log(self) -> "Buffer":
        return self._unary(UnaryOps.LOG)

    def sqrt(self) -> "Buffer":
        return self._unary(UnaryOps.SQRT)

    def rsqrt(self) -> "Buffer":
        return self._unary(UnaryOps.RSQRT)

    def clamp(self, min: int | None = None, max: int | None = None) -> "Buffer":
        return self._unary(UnaryOps.CLAMP, min_val=min, max_val=max)

    def __neg__(self) -> "Buffer":
        return self._unary(UnaryOps.NEG)

    def __pow__(self, val: Scalar) -> "Buffer":
        return self._unary(UnaryOps.POW, val=val)

    # compositions, same formulas as buffer.py:338-362
    def relu(self) -> "Buffer":
        return self.where(inp=self, other=0.0)

    def leaky_relu(self, neg_slope: Scalar = 0.01) -> "Buffer":
        return self.where(inp=self, other=self * neg_slope)

    def sigmoid(self) -> "Buffer":
        e = self.exp()
        return e / (e + 1.0)

    def tanh(self) -> "Buffer":
        p, n = self.exp(), (-self).exp()
        return (p - n) / (p + n)

    def softmax(self, dim: int) -> "Buffer":
        """Fused row softmax (one kernel instead of max, sub, exp, sum, div)."""
        return self._unary(CustomOps.SOFTMAX, dim=dim)

    def softmax_bwd(self, upstream: "Buffer") -> "Buffer":
        """self is a softmax output over the last axis; returns self * (upstream - sum(upstream * self))."""
        return self._like(self._dispatch(CustomOps.SOFTMAX_BWD, y=self, g=upstream))

    def masked_softmax(self, mask: "Buffer", scale: float) -> "Buffer":
        """softmax over the last axis of self * scale with -inf where mask > 0, one kernel."""
        return self._like(self._dispatch(CustomOps.MASKED_SOFTMAX, x=self, mask=mask, scale=scale))

    def masked_softmax_bwd(self, upstream: "Buffer", mask: "Buffer", scale: float) -> "Buffer":
        """self is a masked_softmax output; returns the gradient of its input."""
        return self._like(self._dispatch(CustomOps.MASKED_SOFTMAX_BWD, y=self, g=upstream, mask=mask, scale=scale))

    @staticmethod
    def _attention_kept(p, B: int, n_head: int, T: int) -> tuple:
        """Shape of what a causal attention keeps for its backward pass: the probabilities (B, n_head, T, T), or the
        log-sum-exp of every score row (B, n_head, T) where the runtime's kernels never store the probabilities."""
        nbytes = getattr(p, "nbytes", None)
        return (B, n_head, T) if nbytes is not None and nbytes < 4 * B * n_head * T * T else (B, n_head, T, T)

    def causal_attention(self, k: "Buffer", v: "Buffer", n_head: int, scale: float) -> tuple["Buffer", "Buffer"]:
        """self, k, v: (B, T, C) projections with C = n_head * d.  Returns the context (B, T, C) and the
        attention probabilities (B, n_head, T, T); the heads are read and written in place."""
        B, T, _ = self.shape
        y, p = self._dispatch(CustomOps.CAUSAL_ATTENTION, q=self, k=k, v=v, n_head=n_head, scale=scale)
        return self._like(y), self._like(p, self._attention_kept(p, B, n_head, T))

    def causal_attention_bwd(self, k: "Buffer", v: "Buffer", p: "Buffer", dy: "Buffer", n_head: int,
                             scale: float, y: "Buffer | None" = None) -> tuple["Buffer", "Buffer", "Buffer"]:
        """Gradients of causal_attention for q = self, k, v, each (B, T, C); y: its context, if kept."""
        dq, dk, dv = self._dispatch(CustomOps.CAUSAL_ATTENTION_BWD, q=self, k=k, v=v, p=p, dy=dy, n_head=n_head, scale=scale, y=y)
        return self._like(dq), self._like(dk), self._like(dv)

    def causal_attention_qkv(self, n_head: int, scale: float) -> tuple["Buffer", "Buffer"]:
        """self: (B, T, 3C) with q, k, v side by side per position.  Returns the context (B, T, C) and the
        probabilities (B, n_head, T, T)."""
        B, T, C3 = self.shape
        y, p = self._dispatch(CustomOps.CAUSAL_ATTENTION_QKV, qkv=self, n_head=n_head, scale=scale)
        return self._like(y, (B, T, C3 // 3)), self._like(p, self._attention_kept(p, B, n_head, T))

    def causal_attention_qkv_bwd(self, p: "Buffer", dy: "Buffer", n_head: int, scale: float, y: "Buffer | None" = None) -> "Buffer":
        """Gradient of causal_attention_qkv with respect to self, same (B, T, 3C) layout."""
        return self._like(self._dispatch(CustomOps.CAUSAL_ATTENTION_QKV_BWD, qkv=self, p=p, dy=dy, n_head=n_head, scale=scale, y=y))

    def cached_attention(self, k_store: "Buffer", v_store: "Buffer", n: int, n_head: int, scale: float,
                         hidden: "Buffer | None" = None) -> "Buffer":
        """self: (B, 1, C) query projection; k_store, v_store: (block, B, C) caches of which the first n
        rows take part (minus those `hidden` marks).  Returns the context (B, 1, C)."""
        return self._like(self._dispatch(CustomOps.CACHED_ATTENTION, q=self, k_store=k_store, v_store=v_store, n=n,
                                         n_head=n_head, scale=scale, hidden=hidden))

    def log_softmax(self, dim: int) -> "Buffer":
        return self._unary(CustomOps.LOG_SOFTMAX, dim=dim)

    def log_softmax_gather(self, target: "Buffer") -> tuple["Buffer", "Buffer"]:
        """(log_softmax(self, last axis), its entries at the target columns as (1, N))."""
        lsm, picked = self._dispatch(CustomOps.LOG_SOFTMAX_GATHER, x=self, target=target)
        return self._like(lsm), self._like(picked, (1, self.shape[0]))

    def ce_grad(self, target: "Buffer", upstream: "Buffer", n: float) -> "Buffer":
        """self is a log-softmax; returns ((exp(self) - onehot(target)) * upstream) / n."""
        return self._like(self._dispatch(CustomOps.CE_GRAD, lsm=self, target=target, upstream=upstream, n=n))

    def ce_stats(self, target: "Buffer", negate: bool = False) -> tuple["Buffer", "Buffer", "Buffer"]:
        """self: (N, V) logits.  Returns per row the max, log(sum(exp(x - max))) and the target's
        log-probability (its negative, the row's loss, with negate), each as (1, N) -- the
        cross-entropy forward without a log-softmax tensor."""
        n = self.shape[0]
        m, ls, picked = self._dispatch(CustomOps.CE_STATS, x=self, target=target, negate=negate)
        return self._like(m, (1, n)), self._like(ls, (1, n)), self._like(picked, (1, n))

    def ce_grad_logits(self, m: "Buffer", ls: "Buffer", target: "Buffer", upstream: "Buffer", n: float) -> "Buffer":
        """self: the logits ce_stats saw, m / ls: its row statistics.  Returns
        ((softmax(self) - onehot(target)) * upstream) / n."""
        return self._like(self._dispatch(CustomOps.CE_GRAD_LOGITS, x=self, m=m, ls=ls, target=target,
                                         upstream=upstream, n=n))

    def rmsnorm(self, weight: "Buffer | None", eps: float) -> tuple["Buffer", "Buffer"]:
        """Fused RMSNorm over the last axis; returns (y, r) with r = rsqrt(mean(x^2) + eps)
        per row, kept for the backward pass."""
        y, r = self._dispatch(CustomOps.RMSNORM, x=self, w=weight, eps=eps)
        return self._like(y), self._like(r, (self.numel // max(self.shape[-1], 1),))

    def rmsnorm_bwd(self, weight: "Buffer | None", r: "Buffer", dy: "Buffer",
                    through_mean: bool, plus: "Buffer | None" = None) -> tuple["Buffer", "Buffer | None"]:
        """self is the forward input x; returns (dx, dw) with dw shaped like the weight.  plus: added to dx as it is stored."""
        kw = {"plus": plus} if plus is not None else {}
        if weight is not None and self.device is Device.HIP and PENDING_SUMS:
            kw["partial_dw"] = True             # dw may come back as the partial rows themselves: (pointer, rows)
        dx, dw = self._dispatch(CustomOps.RMSNORM_BWD, x=self, w=weight, r=r, dy=dy, through_mean=through_mean, **kw)
        if dw.__class__ is tuple:
            part, rows = dw
            return self._like(dx), PartialSum.of(self._like(part, (rows, weight.numel)), weight.shape)
        return self._like(dx), (None if dw is None else self._like(dw, weight.shape))

    # ---- selects ----------------------------------------------------------------------------------
    def where(self, inp: "Buffer | Scalar", other: "Buffer | Scalar") -> "Buffer":
        inp = Buffer.from_scalar(inp) if _is_scalar(inp) else inp
        other = Buffer.from_scalar(other) if _is_scalar(other) else other
        return self._like(self._dispatch(UnaryOps.WHERE, cond=self, x=inp, y=other))

    @staticmethod
    def masked_fill(x: "Buffer", mask: "Buffer", val: Scalar) -> "Buffer":
        out_shape = get_broadcast_shape(x.shape, mask.shape)
        return x._like(x._dispatch(UnaryOps.MASKED_FILL, x=x, mask=mask, val=val, out_shape=out_shape),
                       out_shape)

    # ---- cross-entropy and embedding helpers ---------------------------------------------------------
    @staticmethod
    def ce_forward(x: "Buffer", y: "Buffer") -> "Buffer":
        return x._like(x._dispatch(CustomOps.CE_FORWARD, x=x, y=y), (1, x.shape[0]))

    @staticmethod
    def ce_backward(**kwargs) -> None:
        """Same calling convention as buffer.py:397-400 (op and device arrive as kwargs);
        the target device is the one of `x`."""
        kwargs.pop("device", None)
        op = kwargs.pop("op")
        kwargs["x"]._dispatch(op, **kwargs)

    def embedding(self, idx: "Buffer", backward: bool = False, upstream_grad: "Buffer" = None) -> "Buffer":
        if backward:
            return self._like(self._dispatch(CustomOps.EMBEDDING, x=self, idx=idx, out_numel=self.numel,
                                             backward=True, upstream_grad=upstream_grad))
        out_shape = idx.shape + (self.shape[-1],)
        return self._like(self._dispatch(CustomOps.EMBEDDING, x=self, idx=idx, out_numel=prod_(out_shape)),
                          out_shape)

    def adam_step(self, g: "Buffer", m: "Buffer", v: "Buffer", consts: tuple) -> tuple["Buffer", "Buffer", "Buffer"]:
        """One fused Adam update of the parameter `self`; returns new (p, m, v) Buffers."""
        ptrs = self._dispatch(CustomOps.ADAM_STEP, p=self, g=g, m=m, v=v, consts=consts)
        return tuple(self._like(q) for q in ptrs)

    def adam_step_(self, g: "Buffer", m: "Buffer", v: "Buffer", consts: "Buffer") -> None:
        """In-place Adam update of self, m and v with the constants held in device memory."""
        self._dispatch(CustomOps.ADAM_STEP_INPLACE, p=self, g=g, m=m, v=v, consts=consts)

    def freeze(self) -> "Buffer":
        """Marks this Buffer's allocation read-only for the in-place methods (upload_, copy_, row_store_,
        set_values_): for constants that kernels are allowed to recompute instead of reading -- the cached causal
        mask, whose bits the softmax kernels derive from the indices once they recognise its allocation."""
        _frozen[id(self.ptr)] = self.ptr                # (the pointer object is kept, so its id cannot be reused)
        return self

    def _writable(self, what: str) -> None:
        if id(self.ptr) in _frozen:
            raise ValueError(f"{what}: this Buffer is a read-only constant (kernels may compute its values instead of reading them)")

    def row_store_(self, src: "Buffer", idx: "Buffer", also: "tuple[Buffer, Buffer] | None" = None) -> None:
        """self[(int)idx, :] = src, rows being the leading dim of self; idx is a one-element
        Buffer on the same device, read where the kernel runs.  also = (dst2, src2): the same for a
        second destination of the same shape (one launch on the hip device)."""
        self._writable("row_store_")
        rows = self.shape[0]
        width = self.numel // max(rows, 1)
        if src.numel != width or idx.numel != 1 or idx.is_host_scalar:
            raise ValueError(f"row_store_: row of {src.numel} into {self.shape}, index {idx.shape}")
        if also is not None:
            dst2, src2 = also
            if dst2.shape != self.shape or src2.numel != width or dst2.device is not self.device:
                raise ValueError(f"row_store_: second pair {dst2.shape} <- {src2.shape} does not match {self.shape}")
            if self.device is Device.HIP:
                self._dispatch(CustomOps.ROW_STORE, dst=self, src=src, idx=idx, rows=rows, width=width, dst2=dst2, src2=src2)
                return
            dst2.row_store_(src2, idx)
        self._dispatch(CustomOps.ROW_STORE, dst=self, src=src, idx=idx, rows=rows, width=width)

    def embedding_sum(self, pos_table: "Buffer", idx: "Buffer", pos: "Buffer") -> "Buffer":
        """self[idx] + pos_table[pos] for idx (B, T) and pos (T,): (B, T, W), one launch on the hip device."""
        out = self._dispatch(CustomOps.EMBEDDING_SUM, tok_table=self, pos_table=pos_table, idx=idx, pos=pos)
        return Buffer.fresh(out, tuple(idx.shape) + (self.shape[-1],), self.device)

    # ---- the ends of a decoding step (hip) -------------------------------------------------------
    def decode_qkv_row(self, w: "Buffer", gain: "Buffer", eps: float, kc: "Buffer", vc: "Buffer", slot: "Buffer") -> "Buffer":
        """self: one row; w: the stacked (3C, K) q, k, v projection.  Returns q (C,) = the first third of
        rmsnorm(self) @ w^T; the key and value thirds are written to row (int)slot of kc and vc."""
        C = w.shape[-2] // 3
        return Buffer.fresh(self._dispatch(CustomOps.DECODE_QKV_ROW, x=self, w=w, gain=gain, eps=eps, kc=kc, vc=vc, slot=slot),
                            (C,), self.device)

    @staticmethod
    def decode_embed(wte: "Buffer", wpe: "Buffer", slot: "Buffer", T: int, tok: "Buffer | None" = None,
                     seq: "Buffer | None" = None, refpos: bool = False):
        """tok given: (x (1, 1, C), hidden (1, T)) = (wte[tok] + wpe[position of slot], arange(T) > slot).
        seq given: x (1, T, C) = wte[last T tokens of seq up to slot] + wpe[0 .. T - 1]."""
        C = wte.shape[1]
        got = wte._dispatch(CustomOps.DECODE_EMBED, wte=wte, wpe=wpe, slot=slot, T=T, tok=tok, seq=seq, refpos=refpos)
        if seq is not None:
            return Buffer.fresh(got, (1, T, C), wte.device)
        return Buffer.fresh(got[0], (1, 1, C), wte.device), Buffer.fresh(got[1], (1, T), wte.device)

    def decode_next_(self, tok: "Buffer", slot: "Buffer", seq: "Buffer") -> None:
        """self: the logits of the position just computed.  seq[slot + 1] = tok = argmax(self); slot += 1, in place."""
        self._dispatch(CustomOps.DECODE_NEXT, logits=self, tok=tok, slot=slot, seq=seq)

    def decode_sample_(self, u: "Buffer", tok: "Buffer", slot: "Buffer", seq: "Buffer", temperature: float) -> None:
        """self: the logits of the position just computed.  seq[slot + 1] = tok = the token that u[slot] draws from
        softmax(self / temperature) by inversion; slot += 1, in place."""
        self._dispatch(CustomOps.DECODE_SAMPLE, logits=self, u=u, tok=tok, slot=slot, seq=seq, temperature=temperature)

    def sgd_step_(self, g: "Buffer", v: "Buffer | None", lr: float, momentum: float) -> None:
        """In-place SGD update of self (and of the velocity v when momentum is used)."""
        self._dispatch(CustomOps.SGD_STEP_INPLACE, p=self, g=g, v=v, lr=lr, momentum=momentum)

    def set_values_(self, values: tuple) -> None:
        """Writes up to eight floats, given by value, into the first elements of this Buffer with a kernel
        launch (hip): nothing is transferred and the host does not wait."""
        self._writable("set_values_")
        self._dispatch(CustomOps.SET_VALUES, dst=self, values=tuple(values))

    def upload_(self, arr: np.ndarray) -> None:
        """Overwrites this Buffer's memory with `arr` (same element count); the address stays."""
        self._writable("upload_")
        if arr.size != self.numel:
            raise ValueError(f"Buffer size mismatch! Expected {self.numel} elements, got {arr.size}")
        self._dispatch(BufferOps.CREATE, data=arr, into=self)

    def copy_(self, src: "Buffer") -> None:
        """Overwrites this Buffer's memory with the elements of `src` (same count, same
        device) without leaving the device; the address stays."""
        self._writable("copy_")
        if src.numel != self.numel or src.device is not self.device:
            raise ValueError(f"copy_: {src.shape} on {src.device} into {self.shape} on {self.device}")
        self._dispatch(CustomOps.COPY_INTO, dst=self, src=src)

    # ---- binary -----------------------------------------------------------------------------------------
    def _binary_op(self, other: "Buffer", op: BinaryOps) -> "Buffer":
        """x is the operand with more elements and fixes the output shape (buffer.py:402-448).
        A smaller left operand of SUB is handled as -(other - self), as there."""
        check_broadcast(self.shape, other.shape)
        a_host, b_host = self.ptr.__class__ is HostScalar, other.ptr.__class__ is HostScalar
        if a_host and b_host:
            with np.errstate(all="ignore"):
                return self._like(HostScalar(_HOST_BINARY[op](self.ptr.value, other.ptr.value)))
        if self.numel >= other.numel:
            big, small, dev = self, other, (other.device if a_host else self.device)
        else:
            big, small, dev = other, self, (self.device if b_host else other.device)
        out = Buffer.fresh(_dispatch_table[(op, dev)](x=big, y=small), big.shape, dev, self.dtype)
        if op is BinaryOps.SUB and big is not self:
            out = -out
        return out

    @staticmethod
    def _coerce(v) -> "Buffer":
        return v if v.__class__ is Buffer else (Buffer.from_scalar(v) if _is_scalar(v) else v)

    def __add__(self, other) -> "Buffer":
        return self._binary_op(Buffer._coerce(other), BinaryOps.ADD)

    def __sub__(self, other) -> "Buffer":
        return self._binary_op(Buffer._coerce(other), BinaryOps.SUB)

    def __mul__(self, other) -> "Buffer":
        return self._binary_op(Buffer._coerce(other), BinaryOps.MUL)

    def __truediv__(self, other) -> "Buffer":
        other = Buffer._coerce(other)
        if self.numel >= other.numel:
            return self._binary_op(other, BinaryOps.DIV)
        return self._binary_op(other ** -1, BinaryOps.MUL)       # small / big = big**-1 * small

    def __rsub__(self, other: Scalar) -> "Buffer":
        return -(self._binary_op(Buffer._coerce(other), BinaryOps.SUB))

    __radd__ = __add__
    __rmul__ = __mul__

    def __le__(self, other: "Buffer") -> "Buffer":
        out_shape = get_broadcast_shape(self.shape, other.shape)
        return self._like(self._dispatch(BinaryOps.CMP, x=self, y=other, out_shape=out_shape, mode="<="),
                          out_shape)

    def _compare(self, op: BinaryOps, other) -> "Buffer":
        other = Buffer._coerce(other)
        if self.is_host_scalar and other.is_host_scalar:
            return self._like(HostScalar(_HOST_BINARY[op](self.ptr.value, other.ptr.value)))
        return self._like(self._dispatch(op, x=self, y=other))

    def __gt__(self, other) -> "Buffer":
        return self._compare(BinaryOps.GT, other)

    def __ge__(self, other) -> "Buffer":
        return self._compare(BinaryOps.GTE, other)

    def __eq__(self, other) -> "Buffer":  # type: ignore[override]
        return self._compare(BinaryOps.EQT, other)

    __hash__ = object.__hash__

    def __matmul__(self, other: "Buffer") -> "Buffer":
        return self.matmul(other)

    # ---- metadata -----------------------------------------------------------------------------------------
    @property
    def T(self) -> "Buffer":  # noqa: N802
        return self.transpose(0, 1)


# Sums over a leading dim that the hip runtime can leave pending (see PartialSum)
PENDING_SUMS = True
PENDING_SUM_MAX_ROWS = 512          # what one column-sum launch folds; the pending form must mean exactly that launch
# A pending sum keeps all its parts alive until somebody reads it -- rows times the memory of the value, for every weight of
# a model until the optimizer step.  Beyond this many bytes of parts held at once, further sums run at once (one launch each,
# their parts freed) instead of staying pending.
PENDING_SUM_BUDGET_BYTES = int(__import__("os").environ.get("DLGRAD_HIP_PENDING_SUM_BYTES", str(8 << 30)))
_pending_bytes = [0]



class PartialSum(Buffer):
    """A Buffer whose value is `parts.sum(0)` -- the sum over the leading dim of a (rows, *shape)
    Buffer -- and that runs that sum only when somebody asks for its memory.

    The weight gradients of a step are such sums (over the batch for a linear layer, ops.py:287-295;
    over per-wavefront partial rows for an RMSNorm gain), and nothing reads them before the optimizer.
    The one-launch Adam of the hip runtime takes the parts themselves and adds them up as it reads
    the gradient, in the very order the column-sum kernel uses, so the separate launch per weight (a
    quarter of the launches of a char-GPT step) disappears and the bits stay.  Every other reader --
    numpy(), another op, a per-tensor optimizer -- touches `ptr`, which runs the sum then, once."""
    __slots__ = ("parts", "_sum", "offset", "pitch", "whole", "_held")

    @staticmethod
    def of(parts: Buffer, shape: tuple) -> Buffer:
        """The pending sum of `parts` over its leading dim, shaped `shape`; the plain sum where pending
        sums do not apply (another device, too many rows, nothing to add)."""
        rows = parts.shape[0] if parts.ndim else 0
        if (not PENDING_SUMS or parts.device is not Device.HIP or parts.__class__ is PartialSum or not 1 < rows <= PENDING_SUM_MAX_ROWS
                or parts.numel != rows * prod_(shape) or parts.numel == 0
                or _pending_bytes[0] + parts.nbytes > PENDING_SUM_BUDGET_BYTES):
            out = parts.sum(0, keepdim=False)
            return out if out.shape == tuple(shape) else out.reshape(shape)
        b = _new_buffer(PartialSum)
        b.parts, b._sum, b.offset, b.whole = parts, None, 0, None
        _pending_bytes[0] += parts.nbytes
        b._held = parts.nbytes                             # given back when the sum runs or the object goes (__del__)
        b.shape, b.dtype, b.device = tuple(shape), parts.dtype, parts.device
        b.numel, b.stride, b.ndim, b.nbytes = _shape_info(b.shape)
        b.pitch = b.numel                                  # floats from one part to the next
        return b

    def piece(self, start: int, shape: tuple) -> Buffer:
        """Elements [start, start + prod(shape)) of the flat value as a Buffer of their own (the thirds of a
        stacked weight gradient).  While the sum is pending the piece is pending too: it names the same parts,
        `start` floats in, one whole value apart."""
        if self._sum is not None:
            return Buffer(self._sum + start, shape, self.device)
        b = _new_buffer(PartialSum)
        b.parts, b._sum, b.offset, b.pitch, b.whole, b._held = self.parts, None, self.offset + start, self.pitch, self, 0
        b.shape, b.dtype, b.device = tuple(shape), self.dtype, self.device
        b.numel, b.stride, b.ndim, b.nbytes = _shape_info(b.shape)
        return b

    @property
    def pending(self) -> bool:
        return self._sum is None and (self.whole is None or self.whole.pending)

    @property
    def ptr(self):
        if self._sum is None:
            if self.whole is not None:                        # a piece: the whole is summed (once), the piece is a view of it
                self._sum = self.whole.ptr + (self.offset - self.whole.offset)
            else:
                self._sum = self.parts.sum(0, keepdim=False).ptr
            self._drop_parts()
        return self._sum

    def _drop_parts(self) -> None:
        self.parts = None
        if self._held:
            _pending_bytes[0] -= self._held                   # the bytes leave the budget here, once
            self._held = 0

    def __del__(self) -> None:
        held = getattr(self, "_held", 0)
        if held:
            _pending_bytes[0] -= held

    @ptr.setter
    def ptr(self, value) -> None:
        self._sum = value
        self._drop_parts()
