"""Tensor: the user-facing array with reverse-mode autograd.

API and semantics follow dlgrad/tensor.py (OP base class :15-89, Tensor :94-897,
backward :777-809); what is below the Buffer calls is this package's.  Host-memory
assumptions of the reference are replaced by explicit transfers: numpy input is
uploaded (`Buffer.from_numpy`), `numpy()`/`tobytes()` download, `copy_from`
uploads, and a Python float stays on the host until a kernel takes it by value.
"""
from __future__ import annotations

from functools import reduce

import numpy as np

from dlgrad_amd.buffer import Buffer, _is_scalar
from dlgrad_amd.device import Device, as_device
from dlgrad_amd.dtype import DType, Scalar


class OP:
    """Node of the autograd tape: remembers its parents and how to push a gradient back.

    `forward` and `backward` work on Buffers.  `execute` runs forward and wraps the
    result in a Tensor that keeps the node alive only if some parent wants a gradient
    (tensor.py:56-89)."""

    def __init__(self, *data: "Tensor") -> None:
        self.parents: tuple = data
        self.req_grad: list[bool] = [t.requires_grad for t in data]
        self.requires_grad: bool = any(self.req_grad)

    def forward(self, *args, **kwargs):
        raise NotImplementedError(f"forward not implemented for {type(self)}")

    def backward(self, *args, **kwargs):
        raise RuntimeError(f"backward not implemented for {type(self)}")

    def reduce_grad_for_broadcasting(self, grad: Buffer, target_shape: tuple) -> Buffer:
        """Sum `grad` over the dims an operand was broadcast along (tensor.py:38-54):
        leading extra dims first, then every dim where the operand had extent 1."""
        for _ in range(len(grad.shape) - len(target_shape)):
            grad = grad.sum(dim=0)
        for i, (g, t) in enumerate(zip(grad.shape, target_shape)):
            if t == 1 and g > 1:
                grad = grad.sum(dim=i, keepdim=True)
        return grad

    @classmethod
    def execute(cls, *data: "Tensor", **kwargs) -> "Tensor":
        if isinstance(data[0], tuple):
            data = data[0]
        ctx = cls(*data)
        dtype = kwargs.pop("dtype", data[0].dtype)
        device = kwargs.pop("device", data[0].device)
        out = Tensor.__new__(Tensor)
        out.data = ctx.forward(*[t.data for t in data], **kwargs)
        out.data.metadata.dtype = dtype
        out.data.metadata.device = device
        out.requires_grad = ctx.requires_grad
        out._ctx = ctx if ctx.requires_grad else None
        out.grad = None
        return out


import dlgrad_amd.ops as ops  # noqa: E402  (ops subclasses OP, so it is imported after it)


class Tensor:
    def __init__(self, data: "Buffer | np.ndarray | Scalar", requires_grad: bool = False,
                 device: Device | str | None = None) -> None:
        self.requires_grad = requires_grad
        self._ctx: OP | None = None
        self.grad: Tensor | None = None
        if isinstance(data, np.ndarray):
            if data.dtype != np.float32:
                raise ValueError("dlgrad only supports float32 dtype")
            if data.ndim > 4:
                raise ValueError("dlgrad only supports upto 4D tensors")
            self.data = Buffer.from_numpy(data, as_device(device))
        elif isinstance(data, Buffer):
            self.data = data
            if device is not None:
                self.data.metadata.device = as_device(device)
        elif _is_scalar(data):
            self.data = Buffer.from_scalar(float(data))
            self.data.metadata.device = as_device(device)
        else:
            raise ValueError("The data must be of type Buffer, np.ndarray or float")

    # ---- host boundary ----------------------------------------------------------------------
    def numpy(self) -> np.ndarray:
        return self.data.numpy()

    def tobytes(self) -> bytes:
        return self.data.numpy().tobytes()

    def copy_from(self, source_bytes: bytes) -> None:
        if len(source_bytes) != self.nbytes:
            raise ValueError(f"Buffer size mismatch! Expected {self.nbytes} bytes, got {len(source_bytes)}")
        arr = np.frombuffer(source_bytes, dtype=np.float32).reshape(self.shape)
        self.data.ptr = Buffer.from_numpy(arr, self.device).ptr

    def show(self) -> None:
        self.data.show()

    def item(self) -> float:
        return float(self.numpy().reshape(-1)[0])

    # ---- creation ---------------------------------------------------------------------------
    @staticmethod
    def uniform(shape: tuple, device: str | Device | None = Device.CPU, dtype: str | DType | None = DType.FLOAT32,
                low: float = 0.0, high: float = 1.0, requires_grad: bool = False) -> "Tensor":
        return Tensor(Buffer.uniform(shape, device=device, dtype=dtype, low=low, high=high),
                      requires_grad=requires_grad, device=device)

    @staticmethod
    def rand(shape: tuple, device: str | Device | None = Device.CPU, dtype: str | DType | None = DType.FLOAT32,
             requires_grad: bool = False) -> "Tensor":
        return Tensor.uniform(shape, device, dtype, requires_grad=requires_grad)

    @staticmethod
    def full(shape: tuple, fill_value: Scalar, device: Device = Device.CPU, dtype: DType = DType.FLOAT32,
             requires_grad: bool = False) -> "Tensor":
        return Tensor(Buffer.full(shape, fill_value=fill_value, device=device, dtype=dtype),
                      requires_grad=requires_grad, device=device)

    @staticmethod
    def ones(shape: tuple, device: Device = Device.CPU, dtype: DType = DType.FLOAT32,
             requires_grad: bool = False) -> "Tensor":
        return Tensor.full(shape, 1.0, device, dtype, requires_grad)

    @staticmethod
    def ones_like(input: "Tensor", device: Device | None = None, dtype: DType = DType.FLOAT32,
                  requires_grad: bool = False) -> "Tensor":
        return Tensor.full(input.shape, 1.0, device or input.device, dtype, requires_grad)

    @staticmethod
    def zeros_like(input: "Tensor", device: Device | None = None, dtype: DType = DType.FLOAT32,
                   requires_grad: bool = False) -> "Tensor":
        return Tensor.full(input.shape, 0.0, device or input.device, dtype, requires_grad)

    @staticmethod
    def arange(shape: tuple, device: Device = Device.CPU, dtype: DType = DType.FLOAT32,
               requires_grad: bool = False) -> "Tensor":
        return Tensor(Buffer.arange(shape, device=device, dtype=dtype), requires_grad=requires_grad, device=device)

    # ---- binary ---------------------------------------------------------------------------------
    @staticmethod
    def _pair(x, y) -> tuple["Tensor", "Tensor"]:
        if _is_scalar(y):
            y = Tensor(y, device=x.device)
        elif _is_scalar(x):
            x = Tensor(x, device=y.device)
        return x, y

    @staticmethod
    def add(x, y) -> "Tensor":
        return ops.Add.execute(*Tensor._pair(x, y))

    @staticmethod
    def sub(x, y) -> "Tensor":
        return ops.Sub.execute(*Tensor._pair(x, y))

    @staticmethod
    def mul(x, y) -> "Tensor":
        return ops.Mul.execute(*Tensor._pair(x, y))

    @staticmethod
    def div(x, y) -> "Tensor":
        return ops.Div.execute(*Tensor._pair(x, y))

    @staticmethod
    def matmul(x: "Tensor", y: "Tensor") -> "Tensor":
        return ops.MatMul.execute(x, y)

    # ---- layout -----------------------------------------------------------------------------------
    def reshape(self, new_shape: tuple) -> "Tensor":
        return ops.Reshape.execute(self, shape=new_shape)

    def permute(self, order: tuple) -> "Tensor":
        return ops.Permute.execute(self, order=order)

    def transpose(self, dim0: int, dim1: int) -> "Tensor":
        nd = self.ndim
        dim0, dim1 = dim0 % nd, dim1 % nd
        order = list(range(nd))
        order[dim0], order[dim1] = order[dim1], order[dim0]
        return self.permute(tuple(order))

    def squeeze(self, dim: list[int] | int) -> "Tensor":
        return ops.Squeeze.execute(self, dim=dim)

    def unsqueeze(self, dim: list[int] | int) -> "Tensor":
        return ops.Unsqueeze.execute(self, dim=dim)

    # ---- reductions ---------------------------------------------------------------------------------
    def sum(self, dim: int = -1, keepdim: bool = False) -> "Tensor":
        return ops.Sum.execute(self, dim=dim, keepdim=keepdim)

    def mean(self, dim: int = -1, keepdim: bool = False) -> "Tensor":
        return ops.Mean.execute(self, dim=dim, keepdim=keepdim)

    def max(self, dim: int = -1, keepdim: bool = False) -> "Tensor":
        return ops.Max.execute(self, dim=dim, keepdim=keepdim)

    def argmax(self, dim: int = -1) -> "Tensor":
        return Tensor(self.data.argmax(dim))

    # ---- unary / activations ------------------------------------------------------------------------------
    def relu(self) -> "Tensor":
        return ops.Relu.execute(self)

    def leaky_relu(self, neg_slope: Scalar = 0.01) -> "Tensor":
        return ops.LeakyRelu.execute(self, neg_slope=neg_slope)

    def tanh(self) -> "Tensor":
        return ops.Tanh.execute(self)

    def sigmoid(self) -> "Tensor":
        return ops.Sigmoid.execute(self)

    def exp(self) -> "Tensor":
        return ops.Exp.execute(self)

    def log(self) -> "Tensor":
        return ops.Log.execute(self)

    def sqrt(self) -> "Tensor":
        return ops.Sqrt.execute(self)

    def rsqrt(self) -> "Tensor":
        return ops.RSqrt.execute(self)

    def clamp(self, min: int | None = None, max: int | None = None) -> "Tensor":
        return ops.Clamp.execute(self, min=min, max=max)

    def dropout(self, p: Scalar) -> "Tensor":
        return ops.Dropout.execute(self, p=p)

    # ---- compositions --------------------------------------------------------------------------------------
    def linear(self, weight: "Tensor", bias: "Tensor | None") -> "Tensor":
        """self @ weight.T + bias (tensor.py:549-563); weight is (out, in), so every call
        materialises the transpose, as there."""
        if ops.FUSED and self.device is Device.HIP and weight.ndim == 2 and self.ndim >= 2:
            if bias is not None and bias.device is Device.HIP and bias.numel == weight.shape[0] and bias.shape[-1] == bias.numel:
                return ops.LinearNTBias.execute(self, weight, bias)     # the addition happens as the product is stored
            out = ops.LinearNT.execute(self, weight)
        else:
            out = self @ weight.T
        return out + bias if bias is not None else out

    def softmax(self, dim: int = -1) -> "Tensor":
        """exp(x - max) / sum(exp(x - max)) along `dim` (tensor.py:634-649).  Along the last
        axis of a device tensor this is one fused kernel with its own backward node;
        otherwise the reference's five-op composition."""
        if ops.use_fused(self, dim):
            return ops.Softmax.execute(self, dim=dim)
        m = self.max(dim=dim, keepdim=True)
        e = (self - m).exp()
        return e / e.sum(dim=dim, keepdim=True)

    def masked_softmax(self, mask: "Tensor", scale: float = 1.0, dim: int = -1) -> "Tensor":
        """`(self * scale).masked_fill(mask, -inf).softmax(dim)`, the attention chain of
        examples/gpt.py:51-54.  On the hip device, along the last axis, with a mask shaped like
        the trailing dims, this is one kernel forward and one backward (the scores are read and
        the probabilities written once); anywhere else it is that chain, op by op."""
        if ops.use_fused_masked_softmax(self, mask, dim):
            return ops.MaskedSoftmax.execute(self, mask, scale=scale)
        return (self * scale).masked_fill(mask, float("-inf")).softmax(dim=dim)

    def log_softmax(self, dim: int = 1) -> "Tensor":
        m = self - self.max(dim=dim, keepdim=True)
        return m - m.exp().sum(dim=dim, keepdim=True).log()

    def sequential(self, layers: list) -> "Tensor":
        return reduce(lambda inp, layer: layer(inp), layers, self)

    def cross_entropy_loss(self, target: "Tensor") -> "Tensor":
        if _is_scalar(target):
            target = Tensor(target)
        return ops.CrossEntropy.execute(self, target)

    def bcewithlogitsloss(self, target: "Tensor") -> "Tensor":
        if _is_scalar(target):
            target = Tensor(target)
        return ops.BCEWithLogitsLoss.execute(self, target)

    def detach(self) -> "Tensor":
        return Tensor(self.data, requires_grad=False, device=self.device)

    @staticmethod
    def tril(inp: "Tensor", k: Scalar = 0.0) -> "Tensor":
        if _is_scalar(k):
            k = Tensor(k)
        return ops.Tril.execute(inp, k)

    def masked_fill(self, mask: "Tensor", value: Scalar) -> "Tensor":
        return ops.MaskedFill.execute(self, mask, value=value)

    @staticmethod
    def where(cond: "Tensor", inp: "Tensor | Scalar", other: "Tensor | Scalar") -> "Tensor":
        if _is_scalar(inp):
            inp = Tensor(inp)
        if _is_scalar(other):
            other = Tensor(other)
        return ops.Where.execute(cond, inp, other)

    @staticmethod
    def embedding(weight: "Tensor", idx: "Tensor") -> "Tensor":
        return ops.Embedding.execute(weight, idx)

    # ---- autograd -----------------------------------------------------------------------------------------------
    def backward(self) -> None:
        """Reverse pass from a one-element tensor (tensor.py:777-809): depth-first
        topological order of the nodes that carry a ctx, seed gradient 1.0, gradients of a
        tensor used twice are added."""
        assert all(d == 1 for d in self.shape), "backward must be called on a scalar Tensor"
        topo: list[Tensor] = []
        seen: set[int] = set()
        stack: list[tuple[Tensor, bool]] = [(self, False)]
        while stack:                                    # iterative DFS: deep graphs (GPT) stay off the C stack
            node, expanded = stack.pop()
            if expanded:
                topo.append(node)
                continue
            if id(node) in seen or getattr(node, "_ctx", None) is None:
                continue
            seen.add(id(node))
            stack.append((node, True))
            for p in reversed(node._ctx.parents):
                stack.append((p, False))
        self.grad = Tensor(1.0, device=self.device)
        for node in reversed(topo):
            if node.grad is None:
                raise RuntimeError(f"Tensor {node} has no grad")
            ctx = node._ctx
            onto = getattr(ctx, "backward_onto", None)
            if onto is None:
                grads, summed = ctx.backward(node.grad.data), ()
            else:       # an op that can add what a parent has collected so far as it stores that parent's gradient
                have = tuple(p.grad.data if (p.grad is not None and p.requires_grad) else None for p in ctx.parents)
                grads, summed = onto(node.grad.data, have)
            for i, (p, g) in enumerate(zip(ctx.parents, grads)):
                if g is None or not p.requires_grad:
                    continue
                gt = Tensor(g, requires_grad=False, device=g.device)
                p.grad = gt if (p.grad is None or i in summed) else p.grad + gt
        for node in topo:                                # release the tape
            node._ctx = None

    def __getitem__(self, idx: slice) -> "Tensor":
        """Leading-dim slices only, as a view into the same allocation (tensor.py:811-823)."""
        if isinstance(idx, slice) and idx.start is not None and idx.stop is not None and idx.step is None:
            if not 0 <= idx.start <= idx.stop <= self.shape[0]:
                raise IndexError(f"slice {idx.start}:{idx.stop} outside dim of extent {self.shape[0]}")
            view = Buffer(self.data.ptr + idx.start * self.stride[0], (idx.stop - idx.start, *self.shape[1:]),
                          device=self.device, dtype=self.dtype)
            return Tensor(view, requires_grad=self.requires_grad, device=self.device)
        raise ValueError("dlgrad only supports slicing or start, stop are None")

    def __repr__(self) -> str:
        return (f"Tensor<dtype: {self.dtype} device: {self.device}, shape: {self.shape}, ndim: {self.ndim}, "
                f"size: {self.numel * DType.get_n_bytes(self.dtype) / 1e6}mb, requires_grad: {self.requires_grad}>")

    @property
    def T(self) -> "Tensor":  # noqa: N802
        return self.transpose(1, 0)

    def __gt__(self, other: Scalar) -> "Tensor":
        return Tensor(self.data > Tensor(other).data if _is_scalar(other) else self.data > other.data)

    def __ge__(self, other: Scalar) -> "Tensor":
        return Tensor(self.data >= Tensor(other).data if _is_scalar(other) else self.data >= other.data)

    def __eq__(self, other) -> "Tensor":  # type: ignore[override]
        return Tensor(self.data == (Tensor(other).data if _is_scalar(other) else other.data))

    def __hash__(self) -> int:
        return id(self)

    def __add__(self, other) -> "Tensor":
        return Tensor.add(self, other)

    def __radd__(self, other) -> "Tensor":
        return Tensor.add(self, other)

    def __mul__(self, other) -> "Tensor":
        return Tensor.mul(self, other)

    def __rmul__(self, other) -> "Tensor":
        return Tensor.mul(self, other)

    def __sub__(self, other) -> "Tensor":
        return Tensor.sub(self, other)

    def __rsub__(self, other) -> "Tensor":
        return Tensor.sub(Tensor(other, device=self.device), self)

    def __truediv__(self, other) -> "Tensor":
        return Tensor.div(self, other)

    def __pow__(self, val: Scalar) -> "Tensor":
        return ops.Pow.execute(self, y=float(val))

    def __neg__(self) -> "Tensor":
        return Tensor(-self.data, requires_grad=self.requires_grad)

    def __matmul__(self, other: "Tensor") -> "Tensor":
        return Tensor.matmul(self, other)

    @property
    def numel(self) -> int:
        return self.data.numel

    @property
    def shape(self) -> tuple:
        return self.data.shape

    @property
    def stride(self) -> tuple:
        return self.data.stride

    @property
    def ndim(self) -> int:
        return self.data.ndim

    @property
    def dtype(self) -> DType:
        return self.data.dtype

    @property
    def device(self) -> Device:
        return self.data.device

    @property
    def nbytes(self) -> int:
        return self.data.nbytes
