"""GPU parity of the fused RMSNorm kernels.

Forward and backward are compared with (a) the same layer run op by op on the C oracle's
cpu device (the reference's composition, nn/__init__.py:25-41, including its missing
gradient through mean(x^2)), and (b) torch autograd in float64 for the complete gradient
(the kernel's through_mean variant).  Shapes: the reference's own RMSNorm test (4,128,256)
(test/test_gpt.py:88-115), the char-GPT rows (2048 x 128), scaled-GPT rows of 768 floats with
several rows per wavefront, a length that is no multiple of 4, and a row longer than one
float4 per lane.  Tolerances: 1e-5 relative for y (one rsqrt of a 1e-6-accurate mean),
1e-5 of the largest entry for gradients (sums over rows in a different order)."""
import numpy as np
import pytest
import torch

import oracle.cpu_runtime  # noqa: F401  (test infrastructure: registers the cpu device)
from dlgrad_amd import Tensor, nn, ops
from dlgrad_amd.helpers import STRICT_REFERENCE
from dlgrad_amd.runtime import hip
from tests.hip_util import check, dev, require_gpu

pytestmark = pytest.mark.gpu

SHAPES = [(4, 128, 256), (16, 128, 128), (9000, 768), (7, 130), (3, 5, 2048), (5, 4096)]


def _close_abs(got, want, tol, what):
    if hip.COMPILE_ONLY:
        return
    scale = max(float(np.abs(want).max()), 1e-30)
    err = float(np.abs(np.asarray(got, np.float64) - want).max()) / scale
    assert err <= tol, f"{what}: {err:.3e} of the largest entry > {tol:.1e}"


@pytest.mark.parametrize("shape", SHAPES)
def test_fused_layer_matches_the_op_by_op_layer_on_the_cpu_oracle(shape):
    require_gpu()
    if not STRICT_REFERENCE:
        pytest.skip("this comparison is defined for the reference-strict default (the complete gradient is checked against torch)")
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal(shape, dtype=np.float32)
    w = (1 + 0.1 * rng.standard_normal((1, shape[-1]))).astype(np.float32)
    up = rng.standard_normal(shape, dtype=np.float32)
    res = {}
    for device in ("cpu", "hip"):
        norm = nn.RMSNorm(shape[-1], device=device)
        norm.weight.data = Tensor(w, device=device).data
        xt = Tensor(x, device=device, requires_grad=True)
        y = norm(xt)
        if device == "hip":
            assert isinstance(y._ctx, ops.RMSNorm), "the hip layer did not take the fused kernel"
        (y * Tensor(up, device=device)).sum().backward()
        res[device] = (y.numpy(), xt.grad.numpy(), norm.weight.grad.numpy())
    check(res["hip"][0], res["cpu"][0], 1e-5, "y")
    _close_abs(res["hip"][1], res["cpu"][1].astype(np.float64), 1e-5, "dx")
    assert res["hip"][2].shape == (1, shape[-1])
    _close_abs(res["hip"][2], res["cpu"][2].astype(np.float64), 1e-5, "dw")


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("affine", [True, False])
def test_complete_gradient_matches_torch_float64(shape, affine):
    require_gpu()
    rng = np.random.default_rng(sum(shape) + affine)
    x = rng.standard_normal(shape, dtype=np.float32)
    w = (1 + 0.1 * rng.standard_normal((1, shape[-1]))).astype(np.float32)
    up = rng.standard_normal(shape, dtype=np.float32)
    xb, wb = dev(x), (dev(w) if affine else None)
    y, r = xb.rmsnorm(wb, 1e-6)
    dx, dw = xb.rmsnorm_bwd(wb, r, dev(up), through_mean=True)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    ty = tx * torch.rsqrt((tx ** 2).mean(-1, keepdim=True) + 1e-6)
    if affine:
        ty = ty * tw
    (ty * torch.tensor(up, dtype=torch.float64)).sum().backward()
    check(y.numpy(), ty.detach().numpy(), 2e-6, "y vs float64")
    check(r.numpy(), torch.rsqrt((tx ** 2).mean(-1) + 1e-6).detach().numpy().reshape(-1), 1e-6, "r vs float64")
    _close_abs(dx.numpy(), tx.grad.numpy(), 2e-6, "dx vs float64")
    if affine:
        _close_abs(dw.numpy(), tw.grad.numpy(), 1e-5, "dw vs float64")
    else:
        assert dw is None


@pytest.mark.parametrize("shape", SHAPES + [(3, 7, 130)])
@pytest.mark.parametrize("affine,through_mean", [(True, True), (True, False), (False, True)])
def test_gradient_added_on_store_has_the_bits_of_a_separate_addition(shape, affine, through_mean):
    """rmsnorm_bwd(plus=p) stores p + dx: dx is rounded before the addition, so the result equals
    the separate element-wise kernel bit for bit, and dw is untouched."""
    require_gpu()
    rng = np.random.default_rng(sum(shape) + 2 * affine + through_mean)
    x, up, prev = (rng.standard_normal(shape, dtype=np.float32) for _ in range(3))
    w = (1 + 0.1 * rng.standard_normal((1, shape[-1]))).astype(np.float32)
    xb, wb, pb = dev(x), (dev(w) if affine else None), dev(prev)
    _, r = xb.rmsnorm(wb, 1e-6)
    dx, dw = xb.rmsnorm_bwd(wb, r, dev(up), through_mean=through_mean)
    dx2, dw2 = xb.rmsnorm_bwd(wb, r, dev(up), through_mean=through_mean, plus=pb)
    check(dx2.numpy(), (pb + dx).numpy(), 0, "prev + dx")
    if affine:
        check(dw2.numpy(), dw.numpy(), 0, "dw")


def test_a_residual_gradient_is_added_by_the_norm_backward_itself():
    """x feeds a norm and a residual connection: x.grad = g_residual + dx_norm.  The engine hands the
    norm what x has collected so far (OP.backward_onto) instead of running an addition: same bits,
    one kernel fewer."""
    require_gpu()
    from dlgrad_amd import nn, ops
    rng = np.random.default_rng(5)
    x0 = rng.standard_normal((4, 32, 128), dtype=np.float32)
    g0 = rng.standard_normal((4, 32, 128), dtype=np.float32)

    def run(onto):
        x = Tensor(x0, device="hip", requires_grad=True)
        h = x * 1.5                                   # a non-leaf with two consumers
        norm = nn.RMSNorm(128, device="hip")
        if not onto:
            norm_ctx = ops.RMSNorm.backward_onto
            ops.RMSNorm.backward_onto = None
        try:
            before = hip.launch_count
            y = h + norm(h) * 2.0
            (y * Tensor(g0, device="hip")).sum().backward()
            return hip.launch_count - before, x.grad.numpy()
        finally:
            if not onto:
                ops.RMSNorm.backward_onto = norm_ctx

    (n1, a), (n0, b) = run(True), run(False)
    assert n1 == n0 - 1, (n1, n0)
    check(a, b, 0, "x.grad")


def test_rows_that_do_not_fit_fall_back_to_the_composition():
    require_gpu()
    x = np.random.default_rng(3).standard_normal((3, 4100), dtype=np.float32)
    norm = nn.RMSNorm(4100, device="hip")
    y = norm(Tensor(x, device="hip", requires_grad=True))
    assert not isinstance(y._ctx, ops.RMSNorm)
    want = x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6)
    check(y.numpy(), want, 1e-5, "composed RMSNorm on rows of 4100")
