"""Optimizers as Tensor expressions (dlgrad/nn/optim.py:4-70): every update is a handful
of element-wise kernels per parameter and rebinds `param.data` to the new buffer."""
import numpy as np

from dlgrad_amd import ops
from dlgrad_amd.device import Device
from dlgrad_amd.tensor import Tensor


def _rebind(p: Tensor, new) -> None:
    """p.data = new, as the reference's optimizers do -- except for a parameter that is a view into a
    shared allocation (nn.stack_parameters): its new value is copied into place, so it stays where the
    kernels that rely on the stacking expect it."""
    if getattr(p.data.ptr, "base", None) is not None:
        p.data.copy_(new)
    else:
        p.data = new


def _adam_multi(**kw):
    """The hip runtime's update of all parameters by one launch (registered when the runtime is first used)."""
    from dlgrad_amd.dispatch import dispatcher
    from dlgrad_amd.helpers import CustomOps
    return dispatcher.dispatch(CustomOps.ADAM_MULTI_INPLACE, Device.HIP, **kw)


class Optimizer:
    def __init__(self, params: list[Tensor], lr: float = 1e-1) -> None:
        self.params = params
        self.lr = lr

    def step(self) -> None:
        for p in self.params:
            assert p.shape == p.grad.shape, f"The shape of the parameter {p.shape} and its grad {p.grad.shape} do not match"
            _rebind(p, (p - p.grad * self.lr).data)

    def zero_grad(self) -> None:
        for p in self.params:
            p.grad = None


class SGD(Optimizer):
    def __init__(self, params: list[Tensor], lr: float = 1e-3, momentum: float = 0.0,
                 graph_safe: bool | None = None) -> None:
        """graph_safe (hip only): parameters and velocities are updated in place -- sixteen parameters per
        launch -- so a captured step can be replayed.  Same arithmetic, same bits.  None (the default) chooses
        it whenever every parameter is on the hip device and the fused kernels are on; False keeps the
        reference's expression, which rebinds `param.data` to a new buffer per update."""
        super().__init__(params, lr)
        self.momentum = momentum
        self._auto = graph_safe is None       # chosen here: step() follows ops.FUSED if that is switched later
        if graph_safe is None:
            graph_safe = bool(ops.FUSED and params and all(p.device is Device.HIP for p in params))
        self.graph_safe = graph_safe
        self.velocities = {id(p): Tensor.zeros_like(p) for p in params} if momentum else {}

    def step(self) -> None:
        if self.graph_safe and ops.FUSED and self.params and all(p.device is Device.HIP for p in self.params):
            # every parameter in one launch (sixteen at a time): same statements as the launch per parameter
            from dlgrad_amd.runtime.hip import HIP
            live = [p for p in self.params if p.grad is not None]
            for p in live:
                assert p.shape == p.grad.shape, f"The shape of the parameter {p.shape} and its grad {p.grad.shape} do not match"
            HIP.sgd_multi_inplace([(p.data, p.grad.data, self.velocities[id(p)].data if self.momentum != 0 else None) for p in live],
                                  self.lr, self.momentum)
            return
        for p in self.params:
            if p.grad is None:
                continue
            assert p.shape == p.grad.shape, f"The shape of the parameter {p.shape} and its grad {p.grad.shape} do not match"
            if self.graph_safe and (ops.FUSED or not self._auto):
                v = self.velocities[id(p)].data if self.momentum != 0 else None
                p.data.sgd_step_(p.grad.data, v, self.lr, self.momentum)
                continue
            upd = p.grad
            if self.momentum != 0:
                upd = self.velocities[id(p)] * self.momentum + p.grad          # v = mu * v + g
                self.velocities[id(p)] = upd
            _rebind(p, (p - upd * self.lr).data)


class Adam(Optimizer):
    """m = b1 m + (1-b1) g;  v = b2 v + (1-b2) g^2;  p -= lr * m_hat / (sqrt(v_hat) + eps)."""

    def __init__(self, params: list[Tensor], lr: float = 1e-3, betas: tuple[float, float] = (0.9, 0.999),
                 eps: float = 1e-8, graph_safe: bool | None = None) -> None:
        """graph_safe (hip only): parameters and moments are updated in place -- all of them by one
        launch -- and the step-dependent constants live in device memory, so that a captured step can
        be replayed: call advance() before each replay.  Same arithmetic, same bits as the
        per-parameter expressions.  None (the default) chooses it whenever every parameter is on
        the hip device and the fused kernels are on; False keeps one update per parameter that
        rebinds `param.data`, as the reference does."""
        self.params, self.lr, self.eps = params, lr, eps
        self.beta1, self.beta2 = betas
        self.m = {id(p): Tensor.zeros_like(p) for p in params}
        self.v = {id(p): Tensor.zeros_like(p) for p in params}
        self.t = 0
        self._auto = graph_safe is None       # chosen here: step() follows ops.FUSED if that is switched later
        if graph_safe is None:
            graph_safe = bool(ops.FUSED and params and all(p.device is Device.HIP for p in params))
        self.graph_safe = graph_safe
        self.consts = Tensor(np.zeros(8, np.float32), device=params[0].device) if graph_safe else None
        self._table = None                 # device-side address table of the one-launch update
        self._graph_tables: list = []

    def _consts(self) -> tuple:
        c1, c2 = 1.0 - self.beta1 ** self.t, 1.0 - self.beta2 ** self.t
        return (self.beta1, 1.0 - self.beta1, self.beta2, 1.0 - self.beta2, c1, c2, self.eps, self.lr)

    def advance(self) -> None:
        """graph_safe: moves to the next step and writes its constants into device memory with a small
        launch (not capturable: a captured graph reads them from there on every replay)."""
        self.t += 1
        self.consts.data.set_values_(self._consts())

    def step(self) -> None:
        if self.graph_safe and (ops.FUSED or not self._auto):     # (the default follows the switch: with the fused kernels off, the reference's expressions)
            from dlgrad_amd.runtime import hip
            if not hip.capturing():
                self.advance()
            quads = [(p.data, p.grad.data, self.m[id(p)].data, self.v[id(p)].data) for p in self.params
                     if p.grad is not None and p.numel]
            try:
                # every parameter in one launch; the address table is uploaded when the tensors have moved.  A pending
                # sum is handed over as its parts (asking for its ptr would run it)
                self._table = _adam_multi(tensors=quads, consts=self.consts.data, table=self._table)
            except ValueError:                           # some tensor is not 16-byte aligned: one launch per parameter
                pass
            else:
                if self._table["frozen"] and self._table not in self._graph_tables:
                    self._graph_tables.append(self._table)         # a captured graph reads it on every replay
                return
            for pb, gb, mb, vb in quads:
                pb.adam_step_(gb, mb, vb, self.consts.data)
            return
        self.t += 1
        consts = self._consts()
        c1, c2 = consts[4], consts[5]
        for p in self.params:
            k, g = id(p), p.grad
            if ops.FUSED and p.device is Device.HIP:
                # same fp32 operations in the same order as below, in one kernel (bit-identical)
                pb, mb, vb = p.data.adam_step(g.data, self.m[k].data, self.v[k].data, consts)
                _rebind(p, pb)
                self.m[k], self.v[k] = Tensor(mb), Tensor(vb)
                continue
            self.m[k] = ((self.m[k] * self.beta1) + (g * (1.0 - self.beta1))).detach()
            self.v[k] = ((self.v[k] * self.beta2) + ((g ** 2.0) * (1.0 - self.beta2))).detach()
            m_hat, v_hat = self.m[k] / c1, self.v[k] / c2
            _rebind(p, (p - (m_hat / (v_hat.sqrt() + self.eps)) * self.lr).data)
