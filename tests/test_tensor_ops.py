"""Tensor-level forward/backward against PyTorch (CPU, fp32) on both devices.

Follows the reference's own strategy (test/test_ops.py, test/test_backward.py,
test/test_gpt.py, test/test_loss.py, test/test_optim.py): same op families, the same
shape lists and tolerances (atol 1e-6..1e-4, rtol 1e-3..1e-4).  `cpu` runs the graph on the
C restatement (host logic + oracle); `hip` runs it on the MI355X kernels.
"""
import numpy as np
import pytest
import torch

import oracle.cpu_runtime  # noqa: F401  registers the cpu device (test infrastructure)
from dlgrad_amd import Tensor, nn
from dlgrad_amd import helpers
from dlgrad_amd.runtime import hip

DEVICES = [pytest.param("cpu"), pytest.param("hip", marks=pytest.mark.gpu)]
RNG = np.random.default_rng(21)


@pytest.fixture(params=DEVICES)
def device(request):
    if request.param == "hip" and not (hip.available() or hip.COMPILE_ONLY):
        pytest.skip("no HIP device")
    return request.param


def f32(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


def close(got, want, atol=1e-5, rtol=1e-3):
    if hip.COMPILE_ONLY:
        return
    np.testing.assert_allclose(np.asarray(got), np.asarray(want), atol=atol, rtol=rtol)


def both(xs, device, requires_grad=True):
    ts = [Tensor(x, requires_grad=requires_grad, device=device) for x in xs]
    tt = [torch.tensor(x, requires_grad=requires_grad) for x in xs]
    return ts, tt


BCAST = [((2, 3, 4, 5), (2, 3, 4, 5)), ((2, 3, 4, 5), (1, 3, 4, 5)), ((2, 3, 4, 5), (2, 1, 4, 1)),
         ((2, 3, 4, 5), (1, 1, 1, 5)), ((2, 3, 4), (3, 4)), ((2, 3, 4), (1, 1, 4)), ((784, 64), (1, 64)),
         ((784, 64), (784, 1)), ((5, 6), (6,))]


@pytest.mark.parametrize("xs,ys", BCAST)
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_binary_forward_backward(op, xs, ys, device):
    x, y = f32(*xs), f32(*ys) + 3
    f = {"add": lambda a, b: a + b, "sub": lambda a, b: a - b, "mul": lambda a, b: a * b,
         "div": lambda a, b: a / b}[op]
    for swap in (False, True):
        (a, b), (ta, tb) = both((x, y), device)
        out, tout = (f(b, a), f(tb, ta)) if swap else (f(a, b), f(ta, tb))
        close(out.numpy(), tout.detach())
        out.sum().backward()
        tout.sum().backward()
        close(a.grad.numpy(), ta.grad, atol=1e-4)
        close(b.grad.numpy(), tb.grad, atol=1e-4)


def test_scalar_operands(device):
    x = f32(4, 5)
    (a,), (ta,) = both((x,), device)
    out = ((a * 2.0 + 1.0) / 3.0 - 0.5)
    tout = ((ta * 2.0 + 1.0) / 3.0 - 0.5)
    close(out.numpy(), tout.detach())
    close((1.0 - a).numpy(), (1.0 - ta).detach())
    close((2.0 * a).numpy(), (2.0 * ta).detach())
    out.sum().backward()
    tout.sum().backward()
    close(a.grad.numpy(), ta.grad)


@pytest.mark.parametrize("shape", [(4, 7), (3, 4, 5), (2, 3, 4, 5), (128, 65)])
def test_reductions_forward_backward(shape, device):
    x = f32(*shape)
    for d in range(len(shape)):
        for keep in (False, True):
            (a,), (ta,) = both((x,), device)
            s, ts = a.sum(d, keepdim=keep), ta.sum(d, keepdim=keep)
            close(s.numpy(), ts.detach(), atol=1e-4)
            (s * s).sum().backward()
            (ts * ts).sum().backward()
            close(a.grad.numpy(), ta.grad, atol=1e-3)
            (a,), (ta,) = both((x,), device)
            m, tm = a.max(d, keepdim=keep), ta.max(d, keepdim=keep).values
            close(m.numpy(), tm.detach(), atol=0, rtol=0)
            m.sum().backward()
            tm.sum().backward()
            close(a.grad.numpy(), ta.grad)
    (a,), (ta,) = both((x,), device)
    close(a.sum().numpy(), ta.sum().detach(), atol=1e-3)
    close(a.mean().numpy(), ta.mean().detach())
    close(a.max().numpy(), ta.max().detach(), atol=0, rtol=0)
    close(a.mean(len(shape) - 1).numpy(), ta.mean(-1).detach())


def test_mean_backward_is_zero_when_reference_strict(device):
    """cpu.py:252 truncates full()'s fill value to int, so Mean.backward's 1/N becomes 0."""
    (a,), (ta,) = both((f32(6, 8),), device)
    a.mean(1).sum().backward()
    ta.mean(1).sum().backward()
    if helpers.STRICT_REFERENCE:
        close(a.grad.numpy(), np.zeros((6, 8), np.float32), atol=0, rtol=0)
    else:
        close(a.grad.numpy(), ta.grad)


UNARY = [("exp", lambda t: t.exp(), False), ("log", lambda t: t.log(), True), ("sqrt", lambda t: t.sqrt(), True),
         ("rsqrt", lambda t: t.rsqrt(), True), ("relu", lambda t: t.relu(), False),
         ("tanh", lambda t: t.tanh(), False), ("sigmoid", lambda t: t.sigmoid(), False),
         ("pow2", lambda t: t ** 2, False), ("pow3", lambda t: t ** 3, False)]


@pytest.mark.parametrize("name,fn,positive", UNARY)
def test_unary_forward_backward(name, fn, positive, device):
    x = f32(13, 17)
    x = np.abs(x) + np.float32(0.1) if positive else x
    (a,), (ta,) = both((x,), device)
    out, tout = fn(a), fn(ta)
    close(out.numpy(), tout.detach())
    out.sum().backward()
    tout.sum().backward()
    close(a.grad.numpy(), ta.grad, atol=1e-4)


def test_leaky_relu_where_clamp(device):
    x, y = f32(9, 11), f32(9, 11)
    (a, b), (ta, tb) = both((x, y), device)
    close(a.leaky_relu(0.01).numpy(), torch.nn.functional.leaky_relu(ta, 0.01).detach())
    w, tw = Tensor.where(a, a, b), torch.where(ta > 0, ta, tb)
    close(w.numpy(), tw.detach(), atol=0, rtol=0)
    w.sum().backward()
    tw.sum().backward()
    close(b.grad.numpy(), tb.grad, atol=0, rtol=0)
    close(a.clamp(-0.5, 0.5).numpy(), ta.clamp(-0.5, 0.5).detach(), atol=0, rtol=0)
    close((a > 0.0).numpy(), (ta > 0).float(), atol=0, rtol=0)


@pytest.mark.parametrize("xs,ys", [((2, 3), (3, 4)), ((128, 784), (784, 64)), ((4, 5, 7), (4, 7, 3)),
                                   ((4, 5, 7), (7, 3)), ((2, 3, 5, 7), (2, 3, 7, 4)), ((2, 3, 5, 7), (7, 4)),
                                   ((2, 1, 5, 7), (2, 3, 7, 4)), ((4, 6, 50, 20), (4, 6, 20, 10))])
def test_matmul_forward_backward(xs, ys, device):
    (a, b), (ta, tb) = both((f32(*xs), f32(*ys)), device)
    out, tout = a @ b, ta @ tb
    close(out.numpy(), tout.detach(), atol=1e-4)
    out.sum().backward()
    tout.sum().backward()
    close(a.grad.numpy(), ta.grad, atol=1e-3)
    close(b.grad.numpy(), tb.grad, atol=1e-3)


def test_linear_and_transposes(device):
    (x, w, b), (tx, tw, tb) = both((f32(32, 20), f32(8, 20), f32(1, 8)), device)
    out, tout = x.linear(w, b), tx @ tw.T + tb
    close(out.numpy(), tout.detach(), atol=1e-5)
    out.sum().backward()
    tout.sum().backward()
    close(w.grad.numpy(), tw.grad, atol=1e-4)
    close(b.grad.numpy(), tb.grad, atol=1e-4)
    (y,), (ty,) = both((f32(2, 3, 4, 5),), device)
    close(y.transpose(1, 2).numpy(), ty.transpose(1, 2).detach(), atol=0, rtol=0)
    z, tz = y.transpose(2, 3).reshape((2, 3, 20)), ty.transpose(2, 3).reshape(2, 3, 20)
    (z * z).sum().backward()
    (tz * tz).sum().backward()
    close(y.grad.numpy(), ty.grad)


@pytest.mark.parametrize("shape,dim", [((4, 7), 1), ((4, 7), 0), ((2, 3, 8), 2), ((2, 4, 16, 16), 3), ((2, 4, 16, 16), 1)])
def test_softmax_and_log_softmax(shape, dim, device):
    x, g = f32(*shape), f32(*shape)
    (a,), (ta,) = both((x,), device)
    s, ts = a.softmax(dim), torch.softmax(ta, dim)
    close(s.numpy(), ts.detach(), atol=1e-6)
    (s * Tensor(g, device=device)).sum().backward()
    (ts * torch.tensor(g)).sum().backward()
    close(a.grad.numpy(), ta.grad, atol=1e-5)
    (a,), (ta,) = both((x,), device)
    close(a.log_softmax(dim).numpy(), torch.log_softmax(ta, dim).detach(), atol=1e-5)


@pytest.mark.parametrize("T", [32, 128])
def test_causal_mask_softmax(T, device):
    (a,), (ta,) = both((f32(2, 2, T, T),), device)
    mask = Tensor.tril(Tensor.ones((T, T), device=device), k=0.0) == Tensor(0.0)
    out = a.masked_fill(mask, float("-inf")).softmax(3)
    tmask = torch.tril(torch.ones(T, T)) == 0
    tout = torch.softmax(ta.masked_fill(tmask, float("-inf")), 3)
    close(out.numpy(), tout.detach(), atol=1e-6)
    g = f32(2, 2, T, T)
    (out * Tensor(g, device=device)).sum().backward()
    (tout * torch.tensor(g)).sum().backward()
    close(a.grad.numpy(), ta.grad, atol=1e-5)


def test_embedding_forward_backward(device):
    table = f32(100, 32)
    idx = RNG.integers(0, 100, (4, 16))
    w = Tensor(table, requires_grad=True, device=device)
    out = Tensor.embedding(w, Tensor(idx.astype(np.float32), device=device))
    tw = torch.tensor(table, requires_grad=True)
    tout = torch.nn.functional.embedding(torch.tensor(idx), tw)
    close(out.numpy(), tout.detach(), atol=0, rtol=0)
    g = f32(4, 16, 32)
    (out * Tensor(g, device=device)).sum().backward()
    (tout * torch.tensor(g)).sum().backward()
    close(w.grad.numpy(), tw.grad, atol=1e-5)


@pytest.mark.parametrize("shape", [(4, 7), (128, 100), (1000, 1000)])
def test_cross_entropy_sum_forward_mean_backward(shape, device):
    """CrossEntropy.forward returns the SUM of the row losses while its backward is the
    gradient of the MEAN (ops.py:356-357 vs :368)."""
    x = f32(*shape)
    t = RNG.integers(0, shape[1], (shape[0], 1))
    (a,), (ta,) = both((x,), device)
    loss = a.cross_entropy_loss(Tensor(t.astype(np.float32), device=device))
    tl = torch.nn.functional.cross_entropy(ta, torch.tensor(t[:, 0]), reduction="sum")
    close(loss.numpy(), tl.detach(), rtol=1e-4)
    loss.backward()
    (tl / shape[0]).backward()
    close(a.grad.numpy(), ta.grad, atol=1e-6, rtol=1e-4)


@pytest.mark.parametrize("shape", [(4, 7), (128, 100)])
def test_cross_entropy_mean_forward(shape, device):
    """CCrossEntropy (ops.py:372-396): the MEAN of the row losses, which is what torch's default
    reduction gives, and the same gradient as CrossEntropy."""
    from dlgrad_amd import ops
    x = f32(*shape)
    t = RNG.integers(0, shape[1], (shape[0], 1))
    (a,), (ta,) = both((x,), device)
    loss = ops.CCrossEntropy.execute(a, Tensor(t.astype(np.float32), device=device))
    tl = torch.nn.functional.cross_entropy(ta, torch.tensor(t[:, 0]))
    close(loss.numpy().reshape(()), tl.detach(), atol=1e-6, rtol=1e-4)
    loss.backward()
    tl.backward()
    close(a.grad.numpy(), ta.grad, atol=1e-6, rtol=1e-4)


@pytest.mark.parametrize("shape", [(4, 7), (1000, 1000)])
def test_bce_with_logits_forward_backward(shape, device):
    """test/test_loss.py:39-65: mean of the numerically stable BCE-with-logits and its
    gradient (sigmoid(x) - t) / N, against torch."""
    x = RNG.uniform(-1.0, 1.0, shape).astype(np.float32)
    t = RNG.integers(0, 2, shape).astype(np.float32)
    (a,), (ta,) = both((x,), device)
    loss = a.bcewithlogitsloss(Tensor(t, device=device))
    tl = torch.nn.BCEWithLogitsLoss()(ta, torch.tensor(t))
    close(loss.numpy().reshape(()), tl.detach(), atol=1e-6, rtol=1e-4)
    loss.backward()
    tl.backward()
    close(a.grad.numpy(), ta.grad, atol=1e-5, rtol=1e-4)


def test_rmsnorm_forward(device):
    x = f32(4, 128, 256)
    norm = nn.RMSNorm(256, device=device)
    out = norm(Tensor(x, device=device)).numpy()
    tx = torch.tensor(x)
    want = tx * torch.rsqrt((tx ** 2).mean(-1, keepdim=True) + 1e-6)
    close(out, want, atol=1e-5)


@pytest.mark.parametrize("opt_name", ["sgd", "adam"])
def test_optimizers_five_steps(opt_name, device):
    x, w0 = f32(16, 10), f32(4, 10)
    w = Tensor(w0.copy(), requires_grad=True, device=device)
    tw = torch.tensor(w0.copy(), requires_grad=True)
    opt = nn.optim.SGD([w], lr=1e-2) if opt_name == "sgd" else nn.optim.Adam([w], lr=1e-2)
    topt = torch.optim.SGD([tw], lr=1e-2) if opt_name == "sgd" else torch.optim.Adam([tw], lr=1e-2)
    for _ in range(5):
        opt.zero_grad()
        topt.zero_grad()
        loss = ((Tensor(x, device=device) @ w.T) ** 2).sum()
        tloss = ((torch.tensor(x) @ tw.T) ** 2).sum()
        loss.backward()
        tloss.backward()
        opt.step()
        topt.step()
    close(w.numpy(), tw.detach(), atol=1e-4, rtol=1e-3)


def test_slicing_views_and_io(device):
    x = f32(10, 6)
    a = Tensor(x, device=device)
    close(a[2:5].numpy(), x[2:5], atol=0, rtol=0)
    close((a[2:5] + a[5:8]).numpy(), x[2:5] + x[5:8], atol=0, rtol=0)
    assert a.tobytes() == x.tobytes() or hip.COMPILE_ONLY
    b = Tensor(np.zeros((10, 6), np.float32), device=device)
    b.copy_from(x.tobytes())
    close(b.numpy(), x, atol=0, rtol=0)
    with pytest.raises(ValueError):
        Tensor(x.astype(np.float64), device=device)
    with pytest.raises(ValueError):
        b.copy_from(b"123")


def test_dropout_edges_and_tril(device):
    a = Tensor(f32(5, 5), device=device)
    close(a.dropout(1.0).numpy(), np.zeros((5, 5), np.float32), atol=0, rtol=0)
    close(a.dropout(0.0).numpy(), a.numpy(), atol=0, rtol=0)
    close(Tensor.tril(a, 0.0).numpy(), np.tril(a.numpy()), atol=0, rtol=0)
    close(Tensor.tril(a, 1.0).numpy(), np.tril(a.numpy(), 1), atol=0, rtol=0)


def test_the_cached_causal_mask_is_read_only():
    """ops.causal_mask hands out one cached (T, T) Buffer per size and device; the hip softmax kernels recognise
    its allocation and compute its bits from the indices instead of reading them, so writing into it in place
    would silently change nothing they see: the in-place methods refuse."""
    import oracle.cpu_runtime  # noqa: F401
    from dlgrad_amd import ops
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    m = ops.causal_mask(5, Device.CPU)
    np.testing.assert_array_equal(m.numpy(), np.triu(np.ones((5, 5), np.float32), 1))
    with pytest.raises(ValueError, match="read-only"):
        m.upload_(np.zeros((5, 5), np.float32))
    with pytest.raises(ValueError, match="read-only"):
        m.copy_(Buffer.from_numpy(np.zeros((5, 5), np.float32), Device.CPU))
    with pytest.raises(ValueError, match="read-only"):
        m.row_store_(Buffer.from_numpy(np.zeros((5,), np.float32), Device.CPU), Buffer.from_numpy(np.zeros((1,), np.float32), Device.CPU))
    other = Buffer.from_numpy(np.ones((5, 5), np.float32), Device.CPU)
    other.upload_(np.zeros((5, 5), np.float32))                   # ordinary buffers are written as before
    assert not other.numpy().any()
