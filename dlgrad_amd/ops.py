"""Autograd nodes: forward and backward of every Tensor op, written on Buffers.

The formulas, and therefore the sequence of kernels a backward pass issues, are the
ones of dlgrad/ops.py:8-462.  Two things differ on purpose:
  * where the reference reshapes a gradient by mutating Buffer metadata in place
    (`upstream_grad.unsqueeze(dim)`, ops.py:70, :90, :105-110), a reshaped *view* is
    used, so a gradient shared by two consumers is never seen with the wrong shape;
  * `Softmax` is a node of its own when the fused row kernel applies, with the
    closed-form backward y * (g - sum(g * y)).
"""
from __future__ import annotations

import os

from dlgrad_amd.buffer import Buffer, PartialSum
from dlgrad_amd.device import Device
from dlgrad_amd.dtype import Scalar
from dlgrad_amd.helpers import STRICT_REFERENCE, CustomOps, broadcast_shapes, check_broadcast
from dlgrad_amd.tensor import OP

# Fused row kernels (softmax, log-softmax inside cross-entropy) on the hip device.
# Off = the reference's op-by-op compositions, kept as the parity bridge.
FUSED = os.environ.get("DLGRAD_HIP_FUSED", "1") != "0"


def use_fused(t, dim: int) -> bool:
    """dim must name the last axis explicitly: -1 means "all elements" to the reference's
    reductions (helpers.py:204-206), so softmax(dim=-1) is a global softmax there."""
    return FUSED and t.device is Device.HIP and t.ndim >= 1 and dim == t.ndim - 1


def _expand_at(g: Buffer, dim: int, keepdim: bool) -> Buffer:
    """View of a reduced gradient with the reduced dim back as extent 1
    (dim == -1, "all elements", becomes a leading 1 as Buffer.unsqueeze does)."""
    if keepdim:
        return g
    d = 0 if dim == -1 else dim
    shape = list(g.shape)
    shape.insert(d, 1)
    if g.is_host_scalar:
        return g
    return g.reshape(tuple(shape))


# ------------------------------------------------------------------ unary
class Pow(OP):
    def forward(self, x: Buffer, y: float) -> Buffer:
        self.x, self.y = x, y
        return x ** y

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (upstream_grad * ((self.x ** (self.y - 1.0)) * self.y),)      # g * p * x^(p-1)


class Reshape(OP):
    def forward(self, x: Buffer, shape: tuple) -> Buffer:
        self.input_shape = x.shape
        return x.reshape(shape)

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (upstream_grad.reshape(self.input_shape),)


class Permute(OP):
    def forward(self, x: Buffer, order: tuple) -> Buffer:
        self.order = order
        return x.permute(order)

    def backward(self, upstream_grad: Buffer) -> tuple:
        inverse = [0] * len(self.order)
        for i, p in enumerate(self.order):
            inverse[p] = i
        return (upstream_grad.permute(tuple(inverse)),)


class Transpose(OP):
    def forward(self, x: Buffer, dim0: int, dim1: int) -> Buffer:
        self.dims = (dim0, dim1)
        return x.transpose(dim0, dim1)

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (upstream_grad.transpose(self.dims[1], self.dims[0]),)


class _Reduction(OP):
    def _remember(self, x: Buffer, dim: int, keepdim: bool) -> None:
        self.inp_shape, self.device, self.dtype = x.shape, x.device, x.dtype
        self.dim, self.keepdim = dim, keepdim


class Sum(_Reduction):
    def forward(self, x: Buffer, dim: int = -1, keepdim: bool = False) -> Buffer:
        self._remember(x, dim, keepdim)
        return x.sum(dim=dim, keepdim=keepdim)

    def backward(self, upstream_grad: Buffer) -> tuple:
        ones = Buffer.full(shape=self.inp_shape, fill_value=1.0, device=self.device, dtype=self.dtype)
        return (ones * _expand_at(upstream_grad, self.dim, self.keepdim),)


class Mean(_Reduction):
    def forward(self, x: Buffer, dim: int = -1, keepdim: bool = False) -> Buffer:
        self._remember(x, dim, keepdim)
        self.N = x.numel if dim == -1 else x.shape[dim]
        return x.mean(dim=dim, keepdim=keepdim)

    def backward(self, upstream_grad: Buffer) -> tuple:
        # ops.py:86-91.  Buffer.full hands the fill value to the runtime, which truncates
        # it to int when reference-strict (cpu.py:252): 1/N becomes 0 there.
        scale = Buffer.full(self.inp_shape, fill_value=1.0 / self.N, device=self.device, dtype=self.dtype)
        return (scale * _expand_at(upstream_grad, self.dim, self.keepdim),)


class Max(_Reduction):
    def forward(self, x: Buffer, dim: int = -1, keepdim: bool = False) -> Buffer:
        self._remember(x, dim, keepdim)
        self.x = x
        self.out = x.max(dim=dim, keepdim=keepdim)
        return self.out

    def backward(self, upstream_grad: Buffer) -> tuple:
        hit = self.x == _expand_at(self.out, self.dim, self.keepdim)           # 1.0 where x attains the max
        return (hit * _expand_at(upstream_grad, self.dim, self.keepdim),)


class Tril(OP):
    def forward(self, x: Buffer, k: Buffer) -> Buffer:
        H, W = x.shape[0], x.shape[1]                                          # 2-D only (ops.py:116-117)
        rows = Buffer.arange((H, 1), x.device)
        cols = Buffer.arange((1, W), x.device)
        self.mask = cols <= (rows + k)
        return self.mask.where(x, 0.0)

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (self.mask.where(upstream_grad, 0.0),)


class Exp(OP):
    def forward(self, x: Buffer) -> Buffer:
        self.out = x.exp()
        return self.out

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (upstream_grad * self.out,)


class Log(OP):
    def forward(self, x: Buffer) -> Buffer:
        self.x = x
        return x.log()

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (upstream_grad / self.x,)


class Relu(OP):
    def forward(self, x: Buffer) -> Buffer:
        self.out = x.relu()
        return self.out

    def backward(self, upstream_grad: Buffer) -> tuple:
        if FUSED and self.out.device is Device.HIP and upstream_grad.shape == self.out.shape:
            # the 0/1 mask times the gradient as one select: the gradient where out > 0, else 0
            return (self.out.where(inp=upstream_grad, other=0.0),)
        return (self.out.where(inp=1.0, other=0.0) * upstream_grad,)


class LeakyRelu(OP):
    def forward(self, x: Buffer, neg_slope: Scalar = 0.01) -> Buffer:
        self.neg_slope = neg_slope
        self.out = x.leaky_relu(neg_slope=neg_slope)
        return self.out

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (self.out.where(inp=1.0, other=self.neg_slope) * upstream_grad,)


class Sigmoid(OP):
    def forward(self, x: Buffer) -> Buffer:
        self.out = x.sigmoid()
        return self.out

    def backward(self, upstream_grad: Buffer) -> tuple:
        return ((self.out * -(self.out - 1.0)) * upstream_grad,)


class Tanh(OP):
    def forward(self, x: Buffer) -> Buffer:
        self.out = x.tanh()
        return self.out

    def backward(self, upstream_grad: Buffer) -> tuple:
        ones = Buffer.full(self.out.shape, 1.0, self.out.device, self.out.dtype)
        return ((ones - self.out ** 2) * upstream_grad,)


class Sqrt(OP):
    def forward(self, x: Buffer) -> Buffer:
        self.out = x.sqrt()
        return self.out

    def backward(self, grad_output: Buffer) -> tuple:
        return (grad_output / (self.out * 2),)


class RSqrt(OP):
    def forward(self, x: Buffer) -> Buffer:
        self.out = x.rsqrt()
        return self.out

    def backward(self, grad_output: Buffer) -> tuple:
        return (grad_output * (self.out ** 3 * -0.5),)


class Clamp(OP):
    def forward(self, x: Buffer, min: int | None, max: int | None) -> Buffer:
        self.min, self.max = min, max
        return x.clamp(min, max)

    def backward(self, grad_output: Buffer) -> tuple:
        return (grad_output.clamp(self.min, self.max),)                        # as ops.py:204-205


class Squeeze(OP):
    def forward(self, x: Buffer, dim: list[int] | int) -> Buffer:
        self.dim = dim
        x.squeeze(dim)
        return x

    def backward(self, grad_output: Buffer) -> tuple:
        grad_output.unsqueeze(self.dim)
        return (grad_output,)


class Unsqueeze(OP):
    def forward(self, x: Buffer, dim: list[int] | int) -> Buffer:
        self.dim = dim
        x.unsqueeze(dim)
        return x

    def backward(self, grad_output: Buffer) -> tuple:
        grad_output.squeeze(self.dim)
        return (grad_output,)


# ------------------------------------------------------------------ binary
class _Binary(OP):
    def _keep(self, x: Buffer, y: Buffer) -> None:
        check_broadcast(x.shape, y.shape)
        self.x, self.y = x, y

    def _to(self, g: Buffer, which: int) -> Buffer | None:
        if not self.req_grad[which]:
            return None
        return self.reduce_grad_for_broadcasting(g() if callable(g) else g, (self.x, self.y)[which].shape)


class Add(_Binary):
    def forward(self, x: Buffer, y: Buffer) -> Buffer:
        self._keep(x, y)
        return x + y

    def backward(self, upstream_grad: Buffer) -> tuple:
        return self._to(upstream_grad, 0), self._to(upstream_grad, 1)


class Sub(_Binary):
    def forward(self, x: Buffer, y: Buffer) -> Buffer:
        self._keep(x, y)
        return x - y

    def backward(self, upstream_grad: Buffer) -> tuple:
        return self._to(upstream_grad, 0), self._to(lambda: -upstream_grad, 1)


class Mul(_Binary):
    def forward(self, x: Buffer, y: Buffer) -> Buffer:
        self._keep(x, y)
        return x * y

    def backward(self, upstream_grad: Buffer) -> tuple:
        return self._to(lambda: upstream_grad * self.y, 0), self._to(lambda: upstream_grad * self.x, 1)


class Div(_Binary):
    def forward(self, x: Buffer, y: Buffer) -> Buffer:
        self._keep(x, y)
        return x / y

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (self._to(lambda: upstream_grad / self.y, 0),
                self._to(lambda: (-upstream_grad * self.x) / self.y ** 2, 1))


def unbroadcast(grad: Buffer, original_shape: tuple) -> Buffer:
    """Sum a matmul gradient back to an operand that was batch-broadcast (ops.py:287-295).  On the
    hip device the sum over one leading batch dim is left pending (buffer.PartialSum): the one-launch
    optimizer adds the batch entries up as it reads the gradient, any other reader runs the sum."""
    if FUSED and grad.ndim == len(original_shape) + 1 and grad.shape[1:] == tuple(original_shape):
        return PartialSum.of(grad, tuple(original_shape))
    while grad.ndim > len(original_shape):
        grad = grad.sum(0, keepdim=False)
    for i, (g, o) in enumerate(zip(grad.shape, original_shape)):
        if o == 1 and g > 1:
            grad = grad.sum(i, keepdim=True)
    return grad


class MatMul(OP):
    def forward(self, x: Buffer, y: Buffer) -> Buffer:
        self.p1, self.p2, self.out_shape = broadcast_shapes(x.shape, y.shape)
        self.x, self.y = x, y
        return x @ y

    def backward(self, upstream_grad: Buffer) -> tuple:
        """dX = G . Y^T and dY = X^T . G with materialised transposes, then the batch
        broadcast is summed away (ops.py:308-335)."""
        if upstream_grad.shape != self.out_shape:
            upstream_grad = upstream_grad.reshape(self.out_shape)
        xr, yr = self.x.reshape(self.p1), self.y.reshape(self.p2)
        nd = xr.ndim
        if FUSED and upstream_grad.device is Device.HIP:
            # the same two products with the transposed operand read in place: same bits, two
            # permute kernels and two temporaries fewer
            grad_x = upstream_grad.matmul_nt(yr)
            grad_y = xr.matmul_tn(upstream_grad)
        else:
            grad_x = upstream_grad @ yr.transpose(nd - 2, nd - 1)
            grad_y = xr.transpose(nd - 2, nd - 1) @ upstream_grad
        return unbroadcast(grad_x, self.x.shape), unbroadcast(grad_y, self.y.shape)


def product_pair(first: tuple, second: tuple) -> tuple:
    """Two independent products, each (kind, a, b[, epi, e]) as Buffer.matmul_pair takes them: one launch
    on the hip device while the fused kernels are on, two calls otherwise.  Same bits either way."""
    a = first[1]
    if FUSED and a.device is Device.HIP:
        from dlgrad_amd.runtime.hip import HIP
        if HIP.MATMUL_PAIRS:
            return Buffer.matmul_pair(first, second)
    out = []
    for kind, x, y, *rest in (first, second):
        kw = {"epi": rest[0], "e": rest[1]} if rest and rest[0] else {}
        out.append(x.matmul(y, **kw) if kind == "nn" else x.matmul_nt(y, **kw) if kind == "nt" else x.matmul_tn(y))
    return tuple(out)


def tile_norm_applies(x, w, norm) -> bool:
    """Whether the product of the rows of x with w^T can apply the RMSNorm `norm` to x on the way (hip device, fused
    kernels on, a norm with a gain row, rows of at most 128 floats)."""
    if norm is None or norm.weight is None or not FUSED or x.device is not Device.HIP or norm.weight.device is not Device.HIP:
        return False
    from dlgrad_amd.runtime import hip
    how = hip.HIP.NORM_IN_PRODUCT
    if how == "0" or (how != "always" and hip.in_graph()):
        return False
    return w.ndim == 2 and hip.HIP.tile_norm_fits(x.data, w.data if hasattr(w, "data") else w, norm.weight.data)


class _NormInFront:
    """What the ops below share when an RMSNorm sits in front of their first product and is applied inside it:
    they keep x, the gain, the normalised rows (the left operand of the weight gradient) and 1 / rms per row,
    and finish their backward pass with the norm's own backward kernel, which -- like ops.RMSNorm -- can add
    what x has collected so far as it stores dx."""

    def _through_norm(self, dxn: Buffer, plus: Buffer | None) -> tuple:
        return self.x.rmsnorm_bwd(self.gain, self.r, dxn, through_mean=not STRICT_REFERENCE, plus=plus)

    def _plus(self, have: tuple) -> Buffer | None:
        return have[0] if (have[0] is not None and have[0].shape == self.x.shape and have[0].device is self.x.device) else None


class NormLinearNT(OP, _NormInFront):
    """rmsnorm(x, gain) @ W^T for W stored (out, in): RMSNorm followed by LinearNT (the final norm and lm_head of
    examples/gpt.py:100-101) with the normalisation done by the product kernel on its tile of x.  Same values as the
    two nodes, one launch fewer forward."""

    def forward(self, x: Buffer, w: Buffer, gain: Buffer, eps: float = 1e-6) -> Buffer:
        self.x, self.w, self.gain = x, w, gain
        out, self.xn, self.r = x.matmul_nt(w, norm=(gain, eps, True))
        return out

    def _grads(self, upstream_grad: Buffer, plus: Buffer | None) -> tuple:
        dxn, dw = product_pair(("nn", upstream_grad, self.w), ("tn", upstream_grad, self.xn))
        dx, dgain = self._through_norm(unbroadcast(dxn, self.x.shape), plus)
        return dx, unbroadcast(dw, self.w.shape), dgain

    def backward(self, upstream_grad: Buffer) -> tuple:
        return self._grads(upstream_grad, None)

    def backward_onto(self, upstream_grad: Buffer, have: tuple) -> tuple:
        plus = self._plus(have)
        return self._grads(upstream_grad, plus), ((0,) if plus is not None else ())


class LinearNT(OP):
    """x @ W^T for W stored (out, in), the product inside Tensor.linear (tensor.py:549-563),
    with W read in place.  The reference builds it as Transpose -> MatMul, i.e. one permute
    forward and three backward (Y^T, X^T, and the transpose of dW^T back); here
    dX = G @ W and dW = sum over the batch of G^T @ X need none.  Same products, same order
    of additions: bit-identical to that composition -- except for a single row x (decoding), whose
    product runs as one wavefront per output with the k sum split over the lanes (1e-6)."""

    def forward(self, x: Buffer, w: Buffer) -> Buffer:
        self.x, self.w = x, w
        return x.matmul_nt(w)

    def backward(self, upstream_grad: Buffer) -> tuple:
        return _linear_grads(self, upstream_grad)


def _linear_grads(node: OP, upstream_grad: Buffer) -> tuple:
    """(dX, dW) of x @ W^T for a node that kept x and w: one launch for the two products, or only the one that is asked for
    (the input of a network's first layer wants no gradient)."""
    if node.req_grad[0] and node.req_grad[1]:
        grad_x, grad_w = product_pair(("nn", upstream_grad, node.w), ("tn", upstream_grad, node.x))
        return unbroadcast(grad_x, node.x.shape), unbroadcast(grad_w, node.w.shape)
    grad_x = unbroadcast(upstream_grad.matmul(node.w), node.x.shape) if node.req_grad[0] else None
    grad_w = unbroadcast(upstream_grad.matmul_tn(node.x), node.w.shape) if node.req_grad[1] else None
    return grad_x, grad_w


class LinearNTBias(OP):
    """x @ W^T + b with the bias row b (W's row count values) added as the product is stored: the Add node of
    Tensor.linear (tensor.py:549-563) inside LinearNT, one kernel and one pass over the result fewer, same bits.
    Backward: LinearNT's two products, and the column sum that Add's backward gives the bias."""

    def forward(self, x: Buffer, w: Buffer, b: Buffer) -> Buffer:
        self.x, self.w, self.b_shape = x, w, b.shape
        return x.matmul_nt(w, epi="bias", e=b)

    def backward(self, upstream_grad: Buffer) -> tuple:
        grad_b = self.reduce_grad_for_broadcasting(upstream_grad, self.b_shape) if self.req_grad[2] else None    # as Add hands it to the bias
        return (*_linear_grads(self, upstream_grad), grad_b)


class LinearNTAdd(OP):
    """x @ W^T + r with the addition done as the product is stored (r shaped like the result, e.g. the
    residual stream): LinearNT followed by Add, one kernel and one pass over the result fewer, same bits."""

    def forward(self, x: Buffer, w: Buffer, r: Buffer) -> Buffer:
        self.x, self.w = x, w
        return x.matmul_nt(w, epi="add", e=r)

    def backward(self, upstream_grad: Buffer) -> tuple:
        grad_x, grad_w = product_pair(("nn", upstream_grad, self.w), ("tn", upstream_grad, self.x))
        return unbroadcast(grad_x, self.x.shape), unbroadcast(grad_w, self.w.shape), upstream_grad


class MLPRelu(OP):
    """relu(x @ W1^T) @ W2^T (+ r): the feed-forward block of examples/gpt.py:69-78 with the ReLU applied
    as the first product is stored, its backward select applied as the gradient of the hidden layer
    is stored, and the residual added as the second product is stored: the ReLU, its backward and the
    addition no longer run as kernels of their own.  Same values as the op-by-op form: every fused
    step is the same single fp32 operation on the same operands."""

    def forward(self, x: Buffer, w1: Buffer, w2: Buffer, r: Buffer | None = None) -> Buffer:
        self.x, self.w1, self.w2, self.has_r = x, w1, w2, r is not None
        self.h = x.matmul_nt(w1, epi="relu")
        self.gate = self.h                                  # positive where the ReLU let the value through
        return self.h.matmul_nt(w2, epi="add", e=r) if r is not None else self.h.matmul_nt(w2)

    def _products(self, upstream_grad: Buffer, left: Buffer) -> tuple:
        """(gradient of the first product's left operand, dw1, dw2); `left` is that operand."""
        # each gradient of an input travels with the weight gradient that reads the same upstream tensor
        gh, dw2 = product_pair(("nn", upstream_grad, self.w2, "gate", self.gate),      # gradient before the ReLU
                               ("tn", upstream_grad, self.h))
        dx, dw1 = product_pair(("nn", gh, self.w1), ("tn", gh, left))
        return unbroadcast(dx, self.x.shape), unbroadcast(dw1, self.w1.shape), unbroadcast(dw2, self.w2.shape)

    def backward(self, upstream_grad: Buffer) -> tuple:
        dx, dw1, dw2 = self._products(upstream_grad, self.x)
        return (dx, dw1, dw2, upstream_grad) if self.has_r else (dx, dw1, dw2)


class NormMLPRelu(MLPRelu, _NormInFront):
    """x + MLPRelu(rmsnorm(x, gain)): the second half of a transformer block (examples/gpt.py:85) with the norm
    applied inside the first product.  The residual is x itself, so on the way back its gradient -- the upstream
    gradient -- is added by the norm's backward kernel as it stores dx, as it is when the nodes are separate."""

    def forward(self, x: Buffer, w1: Buffer, w2: Buffer, gain: Buffer, eps: float = 1e-6) -> Buffer:
        self.x, self.w1, self.w2, self.gain = x, w1, w2, gain
        self.h, self.xn, self.r = x.matmul_nt(w1, epi="relu", norm=(gain, eps, True))
        self.gate = self.h
        return self.h.matmul_nt(w2, epi="add", e=x)

    def _grads(self, upstream_grad: Buffer, have: Buffer | None) -> tuple:
        dxn, dw1, dw2 = self._products(upstream_grad, self.xn)
        plus = upstream_grad if have is None else have + upstream_grad
        dx, dgain = self._through_norm(dxn, plus)
        return dx, dw1, dw2, dgain

    def backward(self, upstream_grad: Buffer) -> tuple:
        return self._grads(upstream_grad, None)

    def backward_onto(self, upstream_grad: Buffer, have: tuple) -> tuple:
        plus = self._plus(have)
        return self._grads(upstream_grad, plus), ((0,) if plus is not None else ())


def use_fused_epilogues(x, *weights) -> bool:
    return FUSED and x.device is Device.HIP and x.ndim >= 2 and x.numel > 0 and \
        all(w.ndim == 2 and w.device is Device.HIP for w in weights)


class Softmax(OP):
    """Fused forward along the last axis; backward dx = y * (g - sum(g * y, last))."""

    def forward(self, x: Buffer, dim: int) -> Buffer:
        self.out = x.softmax(x.ndim - 1)
        return self.out

    def backward(self, upstream_grad: Buffer) -> tuple:
        from dlgrad_amd.runtime.hip import HIP
        if FUSED and self.out.device is Device.HIP and HIP.softmax_bwd_fits(self.out, upstream_grad):
            return (self.out.softmax_bwd(upstream_grad),)
        gy = upstream_grad * self.out
        return (gy - self.out * gy.sum(dim=self.out.ndim - 1, keepdim=True),)


def use_fused_masked_softmax(x, mask, dim: int) -> bool:
    if not (use_fused(x, dim) and mask.device is Device.HIP):
        return False
    from dlgrad_amd.runtime.hip import HIP
    return HIP.masked_softmax_fits(x.data, mask.data)


class MaskedSoftmax(OP):
    """softmax(masked_fill(x * scale, mask, -inf)) along the last axis as one forward and one
    backward kernel; the values and gradients are those of the three-op chain."""

    def forward(self, x: Buffer, mask: Buffer, scale: float) -> Buffer:
        self.mask, self.scale = mask, scale
        self.out = x.masked_softmax(mask, scale)
        return self.out

    def backward(self, upstream_grad: Buffer) -> tuple:
        from dlgrad_amd.runtime.hip import HIP
        if HIP.softmax_bwd_fits(self.out, upstream_grad):
            return self.out.masked_softmax_bwd(upstream_grad, self.mask, self.scale), None
        gy = upstream_grad * self.out
        g = gy - self.out * gy.sum(dim=self.out.ndim - 1, keepdim=True)
        return Buffer.masked_fill(x=g, mask=self.mask, val=0.0) * self.scale, None


_causal_masks: dict = {}


def causal_mask(T: int, device) -> Buffer:
    """(T, T) of 1.0 where column > row (attention not allowed), else 0.0; built once per size
    and device: what `Tensor.tril(Tensor.ones((T, T))) == 0` gives (examples/gpt.py:52-53)."""
    key = (T, device)
    if key not in _causal_masks:
        allowed = Buffer.arange((1, T), device) <= Buffer.arange((T, 1), device)
        _causal_masks[key] = (allowed == 0.0).freeze()      # read-only: the hip softmax kernels compute these bits instead of reading them
    return _causal_masks[key]


def use_fused_causal_attention(q, k, v) -> bool:
    if not (FUSED and q.device is Device.HIP and k.device is Device.HIP and v.device is Device.HIP):
        return False
    if not (q.ndim == k.ndim == v.ndim and q.ndim >= 2 and q.shape == k.shape and q.shape[:-1] == v.shape[:-1]):
        return False
    from dlgrad_amd.runtime.hip import HIP
    return HIP.causal_softmax_fits(q.shape[-2])


class CausalAttention(OP):
    """softmax(mask(q k^T * scale)) v for q, k (.., T, d) and v (.., T, dv) with the causal mask,
    built from the same kernels as the op-by-op chain of examples/gpt.py:50-55 (a product, the
    scaled masked softmax, a product) and giving the same bits, but knowing the structure:
    k is read in place instead of being transposed first; score tiles that lie entirely
    above the diagonal are not computed (the softmax never reads them); products with the
    probabilities, or with their gradient, stop or start at the diagonal, because everything
    beyond it is an exact zero.  Backward likewise.  Only the probabilities are kept."""

    def forward(self, q: Buffer, k: Buffer, v: Buffer, scale: float) -> Buffer:
        self.q, self.k, self.v, self.scale = q, k, v, scale
        self.mask = causal_mask(q.shape[-2], q.device)
        scores = q.matmul_nt(k, tri="out_lower")
        self.p = scores.masked_softmax(self.mask, scale)
        return self.p.matmul(v, tri="a_lower")

    def backward(self, upstream_grad: Buffer) -> tuple:
        dp = upstream_grad.matmul_nt(self.v, tri="out_lower")
        dv = self.p.matmul_tn(upstream_grad, tri="at_lower")
        ds = self.p.masked_softmax_bwd(dp, self.mask, self.scale)
        dq = ds.matmul(self.k, tri="a_lower")
        dk = ds.matmul_tn(self.q, tri="at_lower")
        return dq, dk, dv


def softmax_row_fits(n: int) -> bool:
    """Whether a row of n scores fits the register-resident masked softmax kernels."""
    from dlgrad_amd.runtime.hip import HIP
    return HIP.causal_softmax_fits(n)


def use_fused_attention_heads(q, k, v, n_head: int) -> bool:
    if not (FUSED and q.device is Device.HIP and k.device is Device.HIP and v.device is Device.HIP):
        return False
    if not (q.ndim == 3 and q.shape == k.shape == v.shape and n_head > 0 and q.shape[2] % n_head == 0 and q.numel):
        return False
    from dlgrad_amd.runtime.hip import HIP
    return HIP.causal_softmax_fits(q.shape[1])


class CausalAttentionHeads(OP):
    """CausalAttention for the (B, T, n_head * d) projections themselves: the products read each head
    where it lies (row pitch n_head * d) and write the context and the three gradients in the same
    layout, so the head split and merge of examples/gpt.py:46-48,57 -- four transposes forward,
    four backward -- never run.  Same kernels, same additions in the same order: the values are
    those of the chain with materialised transposes, bit for bit."""

    def forward(self, q: Buffer, k: Buffer, v: Buffer, n_head: int, scale: float) -> Buffer:
        self.q, self.k, self.v, self.n_head, self.scale = q, k, v, n_head, scale
        self.y, self.p = q.causal_attention(k, v, n_head, scale)
        return self.y

    def backward(self, upstream_grad: Buffer) -> tuple:
        return self.q.causal_attention_bwd(self.k, self.v, self.p, upstream_grad, self.n_head, self.scale, self.y)


def stacked(wq, wk, wv) -> bool:
    """Whether three equal (C, C) weights lie back to back in one allocation, in this order, so that
    together they are one (3C, C) matrix (nn.stack_parameters arranges that)."""
    if not (wq.ndim == 2 and wq.shape == wk.shape == wv.shape and wq.device is Device.HIP):
        return False
    step = 4 * wq.numel
    a = [getattr(w.data.ptr, "addr", None) for w in (wq, wk, wv)]
    return None not in a and a[1] == a[0] + step and a[2] == a[1] + step


def use_fused_qkv_attention(x, wq, wk, wv, n_head: int) -> bool:
    if not (FUSED and x.device is Device.HIP and x.ndim == 3 and x.numel and n_head > 0):
        return False
    C = x.shape[2]
    if wq.shape != (C, C) or C % n_head or not stacked(wq, wk, wv):
        return False
    return softmax_row_fits(x.shape[1])


class SelfAttentionQKV(OP):
    """The three projections and the causal attention of examples/gpt.py:45-57 for weights that are
    stacked in memory: one product x W^T with W = [Wq; Wk; Wv] gives q, k, v side by side, the
    attention kernels read their heads there (row pitch 3C), and backward is one product for dx
    (K = 3C), one for the stacked dW and the attention gradients written into one (B, T, 3C) buffer.
    Per layer 3 + 6 products and two gradient additions become 1 + 2.  q, k, v, the context and
    the weight gradients have the bits of the separate products; dx adds its 3C terms in one
    accumulator instead of three partial sums, so it differs from them by rounding."""

    def forward(self, x: Buffer, wq: Buffer, wk: Buffer, wv: Buffer, gain: Buffer | None = None, n_head: int = 1,
                scale: float = 1.0, eps: float = 1e-6) -> Buffer:
        """gain: the gain row of an RMSNorm that sits in front of the projection and is applied inside it."""
        C = wq.shape[0]
        self.x, self.n_head, self.scale, self.gain = x, n_head, scale, gain
        self.w = Buffer(wq.ptr, (3 * C, C), x.device)                    # the three matrices as one
        if gain is None:
            self.qkv, self.left = x.matmul_nt(self.w), x
        else:
            self.qkv, self.left, self.r = x.matmul_nt(self.w, norm=(gain, eps, True))
        self.y, self.p = self.qkv.causal_attention_qkv(n_head, scale)
        return self.y

    def _grads(self, upstream_grad: Buffer, plus: Buffer | None) -> tuple:
        C = self.w.shape[1]
        g = self.qkv.causal_attention_qkv_bwd(self.p, upstream_grad, self.n_head, self.scale, self.y)     # (B, T, 3C)
        dx, dw = product_pair(("nn", g, self.w), ("tn", g, self.left))
        dw = unbroadcast(dw, self.w.shape)                                                        # (3C, C)
        if dw.__class__ is PartialSum:
            part = lambda i: dw.piece(i * C * C, (C, C))                                          # noqa: E731  (stays pending)
        else:
            part = lambda i: Buffer(dw.ptr + i * C * C, (C, C), dw.device)                        # noqa: E731
        if self.gain is None:
            return dx, part(0), part(1), part(2)
        dx, dgain = _NormInFront._through_norm(self, dx, plus)
        return dx, part(0), part(1), part(2), dgain

    def backward(self, upstream_grad: Buffer) -> tuple:
        return self._grads(upstream_grad, None)

    def backward_onto(self, upstream_grad: Buffer, have: tuple) -> tuple:
        plus = _NormInFront._plus(self, have) if self.gain is not None else None
        return self._grads(upstream_grad, plus), ((0,) if plus is not None else ())


def use_fused_rmsnorm(x, weight) -> bool:
    if not (FUSED and x.device is Device.HIP):
        return False
    from dlgrad_amd.runtime.hip import HIP
    return HIP.rmsnorm_fits(x.data, None if weight is None else weight.data)


class RMSNorm(OP):
    """(x * rsqrt(mean(x^2, last) + eps)) * weight as one forward and one backward kernel
    (plus the column sum that finishes dw).  The gradient through mean(x^2) is dropped when
    reference-strict, as the reference's Mean.backward drops it (ops.py:86-91 with the
    int-truncated fill of cpu.py:252)."""

    def forward(self, x: Buffer, weight: Buffer | None = None, eps: float = 1e-6) -> Buffer:
        self.x, self.weight = x, weight
        y, self.r = x.rmsnorm(weight, eps)
        return y

    def _grads(self, upstream_grad: Buffer, plus: Buffer | None) -> tuple:
        dx, dw = self.x.rmsnorm_bwd(self.weight, self.r, upstream_grad, through_mean=not STRICT_REFERENCE, plus=plus)
        return (dx,) if self.weight is None else (dx, dw)

    def backward(self, upstream_grad: Buffer) -> tuple:
        return self._grads(upstream_grad, None)

    def backward_onto(self, upstream_grad: Buffer, have: tuple) -> tuple:
        """have[0]: the gradient x has collected so far (the residual route around the norm), or None.
        It is added as dx is stored, and parent 0 is reported as already summed."""
        plus = have[0] if (have[0] is not None and have[0].shape == self.x.shape and have[0].device is self.x.device) else None
        return self._grads(upstream_grad, plus), ((0,) if plus is not None else ())


class CrossEntropy(OP):
    def forward(self, logits: Buffer, target: Buffer, dim: int = 1) -> Buffer:
        """log-softmax, gather of the target log-probs, and -SUM over rows -- not the mean
        (ops.py:338-357); backward nevertheless scales by 1/N (ops.py:359-370).
        On the hip device the (N, V) log-softmax is never stored: the forward keeps two numbers
        per row (max and log-sum) and the backward rebuilds each entry from the logits, which the
        tape holds anyway -- one read of the logits forward, one read and one write backward."""
        assert logits.shape[0] == target.shape[0]
        self.target = target
        self.N = float(logits.shape[0])
        self.fused = FUSED and logits.device is Device.HIP and logits.ndim == 2 and dim == 1
        self.stats = None
        if self.fused:
            from dlgrad_amd.runtime.hip import HIP
            if HIP.ce_stats_fits(logits):
                m, ls, row_loss = logits.ce_stats(target, negate=True)
                self.logits, self.stats = logits, (m, ls)
                return self._total(row_loss)                # = -(sum of the picked log-probs), bit for bit
            else:                                           # more than 2^31 elements
                self.log_softmax, picked = logits.log_softmax_gather(target)
        else:
            shifted = logits - logits.max(dim=dim, keepdim=True)
            self.log_softmax = shifted - shifted.exp().sum(dim=dim, keepdim=True).log()
            picked = Buffer.ce_forward(self.log_softmax, self.target)
        return -self._total(picked)

    @staticmethod
    def _total(rows: Buffer) -> Buffer:
        return rows.sum()

    def backward(self, upstream_grad: Buffer) -> tuple:
        if self.stats is not None:
            return (self.logits.ce_grad_logits(*self.stats, self.target, upstream_grad, self.N),)
        if self.fused:
            return (self.log_softmax.ce_grad(self.target, upstream_grad, self.N),)
        probs = self.log_softmax.exp()
        Buffer.ce_backward(op=CustomOps.CE_BACKWARD, device=probs.device, x=probs, target=self.target)   # p - onehot
        return ((probs * upstream_grad) / self.N,)


class CCrossEntropy(CrossEntropy):
    """The mean-reduced form (ops.py:372-396): -MEAN of the picked log-probs, with CrossEntropy's backward
    (which divides by the number of rows either way).  No Tensor method reaches it in the reference."""

    @staticmethod
    def _total(rows: Buffer) -> Buffer:
        return rows.mean()                                  # (-s) / N and -(s / N) are the same bits


class BCEWithLogitsLoss(OP):
    def forward(self, probs: Buffer, target: Buffer) -> Buffer:
        assert probs.shape == target.shape, f"shape mismatch {probs.shape} vs {target.shape}"
        self.probs, self.target = probs, target
        m = (-probs).clamp(min=0)
        loss = ((1.0 - target) * probs) + m + ((-m).exp() + (-(probs + m)).exp()).log()
        return loss.mean()

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (((self.probs.sigmoid() - self.target) * upstream_grad) / float(self.probs.numel),)


class Embedding(OP):
    def forward(self, weight: Buffer, idx: Buffer) -> Buffer:
        self.weight, self.idx = weight, idx
        return weight.embedding(idx)

    def backward(self, upstream_grad: Buffer) -> tuple:
        return (self.weight.embedding(self.idx, backward=True, upstream_grad=upstream_grad),)


class EmbeddingSum(OP):
    """tok_table[idx] + pos_table[pos] for idx (B, T) and pos (T,): the input of a transformer (examples/gpt.py:96-98:
    two Embedding nodes and an Add) as one node and, on the hip device, one launch.  Backward: what those three
    nodes do -- the scatter-add of the upstream rows into the token table, the sum over the batch that Add's
    backward gives its broadcast operand, and the scatter-add of that into the position table."""

    def forward(self, tok_table: Buffer, pos_table: Buffer, idx: Buffer, pos: Buffer) -> Buffer:
        self.tok_table, self.pos_table, self.idx, self.pos = tok_table, pos_table, idx, pos
        return tok_table.embedding_sum(pos_table, idx, pos)

    def backward(self, upstream_grad: Buffer) -> tuple:
        g_tok = g_pos = None
        if self.req_grad[0]:
            g_tok = self.tok_table.embedding(self.idx, backward=True, upstream_grad=upstream_grad)
        if self.req_grad[1]:
            rows = self.reduce_grad_for_broadcasting(upstream_grad, tuple(self.pos.shape) + (self.pos_table.shape[-1],))
            g_pos = self.pos_table.embedding(self.pos, backward=True, upstream_grad=rows)
        return g_tok, g_pos, None, None


class Where(OP):
    def forward(self, cond: Buffer, inp: Buffer, other: Buffer) -> Buffer:
        self.cond = cond
        return cond.where(inp, other)

    def backward(self, upstream_grad: Buffer) -> tuple:
        return None, self.cond.where(upstream_grad, 0.0), self.cond.where(0.0, upstream_grad)


class MaskedFill(OP):
    def forward(self, data: Buffer, mask: Buffer, value: Scalar) -> Buffer:
        self.mask = mask
        return Buffer.masked_fill(x=data, mask=mask, val=value)

    def backward(self, upstream_grad: Buffer) -> tuple:
        return Buffer.masked_fill(x=upstream_grad, mask=self.mask, val=0.0), None, None


class Dropout(OP):
    def forward(self, x: Buffer, p: Scalar) -> Buffer:
        self.p = p
        if p == 1.0:
            return Buffer.full(x.shape, 0.0, x.device, x.dtype)
        if p == 0.0:
            return x
        self.mask = Buffer.uniform(x.shape, x.device, x.dtype, low=0.0, high=1.0) >= p
        self.scale = 1.0 / (1.0 - p)
        return self.mask.where(x, 0.0) * self.scale

    def backward(self, upstream_grad: Buffer) -> tuple:
        if self.p == 1.0:
            return (Buffer.full(upstream_grad.shape, 0.0, upstream_grad.device, upstream_grad.dtype),)
        if self.p == 0.0:
            return (upstream_grad,)
        return (self.mask.where(upstream_grad, 0.0) * self.scale,)
