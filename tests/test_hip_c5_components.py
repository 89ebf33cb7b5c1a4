"""GPU parity at the real shapes of the scaled-GPT config: embedding gather / scatter-add on a
50304 x 768 table with Zipf(1.1) ids, softmax over 98304 rows of 1024, fused cross-entropy
forward + backward on (8192, 50304).

Where the C oracle would take minutes the checks are size-independent properties plus exact
comparison on a slice: gathers bit-exact against numpy indexing; scatter-add against
np.add.at in float64 (1e-5 of the largest entry; atomics reorder the additions); softmax rows
sum to 1 and a slice matches the oracle's five-kernel composition (2e-6); cross-entropy loss
against a float64 log-sum-exp (1e-5) and gradient rows against (softmax - onehot)/N (1e-4 of
the largest entry), every gradient row summing to ~0."""
import numpy as np
import pytest

from dlgrad_amd import Tensor
from dlgrad_amd.runtime import hip
from oracle import cpu_runtime, cref  # noqa: F401  (registers the CPU device the chain is checked against)
from tests.hip_util import check, dev, require_gpu

pytestmark = pytest.mark.gpu
V, W, NTOK = 50304, 768, 8192


def zipf_ids(rng, n, vocab, s=1.1):
    ids = rng.zipf(s, n) - 1
    while (bad := ids >= vocab).any():          # rejection keeps the distribution's shape
        ids[bad] = rng.zipf(s, int(bad.sum())) - 1
    return ids.astype(np.float32)


def test_embedding_gather_and_scatter_add_on_the_50304x768_table():
    require_gpu()
    rng = np.random.default_rng(50)
    table = rng.standard_normal((V, W), dtype=np.float32)
    idx = zipf_ids(rng, NTOK, V).reshape(8, 1024)
    assert hip.COMPILE_ONLY or (idx == 0).sum() > 500          # heavy collisions on the smallest ids
    t = dev(table)
    check(t.embedding(dev(idx)).numpy(), table[idx.astype(np.int64)], 0, "gather 8192 x 768")
    # ids at the top of the table: (int)(idx * 768) must stay exact there (50303 * 768 < 2**26, multiple of 256)
    top = np.array([V - 1, V - 2, 21846, 21845, 0], np.float32)
    check(t.embedding(dev(top)).numpy(), table[top.astype(np.int64)], 0, "gather top ids")
    g = rng.standard_normal((8, 1024, W), dtype=np.float32)
    got = t.embedding(dev(idx), backward=True, upstream_grad=dev(g)).numpy()
    if hip.COMPILE_ONLY:
        return
    want = np.zeros((V, W), np.float64)
    np.add.at(want, idx.astype(np.int64).ravel(), g.reshape(-1, W).astype(np.float64))
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    untouched = np.ones(V, bool)
    untouched[idx.astype(np.int64).ravel()] = False
    assert not got[untouched].any()                              # rows nobody indexed stay exactly zero
    # the integer-index C oracle agrees too (it is the documented stand-in for the reference's float index)
    np.testing.assert_allclose(got, cref.embedding_backward((V, W), idx, g), rtol=0, atol=1e-5 * np.abs(want).max())


def test_softmax_over_98304_rows_of_1024():
    require_gpu()
    rng = np.random.default_rng(51)
    R, L = 8 * 12 * 1024, 1024
    x = rng.standard_normal((R, L), dtype=np.float32) * 2
    x[5, 10:] = -np.inf                                         # a causally masked row: exact zeros expected
    p = dev(x).softmax(1).numpy()
    if hip.COMPILE_ONLY:
        return
    np.testing.assert_allclose(p.sum(1, dtype=np.float64), 1.0, atol=2e-6)
    assert (p[5, 10:] == 0).all()
    for sl in (slice(0, 256), slice(R - 256, R)):
        xs = x[sl]
        m = cref.reduce("max", xs, 1)[:, None]
        e = cref.unary("exp", cref.binary("sub", xs, m))
        check(p[sl], cref.binary("div", e, cref.reduce("sum", e, 1)[:, None]), 2e-6, "softmax slice")


def test_cross_entropy_forward_backward_on_8192x50304():
    require_gpu()
    rng = np.random.default_rng(52)
    logits = rng.standard_normal((NTOK, V), dtype=np.float32)
    tgt = zipf_ids(rng, NTOK, V).reshape(NTOK, 1)
    a = Tensor(logits, requires_grad=True, device="hip")
    loss = a.cross_entropy_loss(Tensor(tgt, device="hip"))
    loss.backward()
    got_loss, grad = float(loss.numpy()), a.grad.numpy()
    if hip.COMPILE_ONLY:
        return
    t = tgt[:, 0].astype(np.int64)
    want_loss, rows = 0.0, np.arange(NTOK)
    for s in range(0, NTOK, 1024):                                # float64 log-sum-exp in chunks
        z = logits[s:s + 1024].astype(np.float64)
        lse = np.log(np.exp(z - z.max(1, keepdims=True)).sum(1)) + z.max(1)
        want_loss += float((lse - z[np.arange(z.shape[0]), t[s:s + 1024]]).sum())
    assert abs(got_loss - want_loss) <= 1e-5 * abs(want_loss)    # forward returns the SUM (ops.py:357)
    sub = rows[::128]
    z = logits[sub].astype(np.float64)
    sm = np.exp(z - z.max(1, keepdims=True))
    sm /= sm.sum(1, keepdims=True)
    sm[np.arange(len(sub)), t[sub]] -= 1
    want = sm / NTOK
    assert np.abs(grad[sub] - want).max() <= 1e-4 * np.abs(want).max()
    assert np.abs(grad.sum(1, dtype=np.float64)).max() <= 1e-6   # each row of softmax - onehot sums to 0


@pytest.mark.parametrize("R,L", [(8 * 12 * 1024, 1024), (8192, 128), (300, 130), (64, 4096)])
def test_fused_softmax_backward_rows(R, L):
    """dx = y (g - sum(g y)): against float64 on a slice, the op-by-op expression on the C oracle's
    kernels on the same slice (1e-5 of the largest entry), and the identity sum(dx) = 0 per row
    (softmax rows sum to 1) over the whole tensor."""
    require_gpu()
    rng = np.random.default_rng(53)
    x = rng.standard_normal((R, L), dtype=np.float32) * 2
    g = rng.standard_normal((R, L), dtype=np.float32)
    y = dev(x).softmax(1)
    dx = y.softmax_bwd(dev(g)).numpy()
    if hip.COMPILE_ONLY:
        return
    yh = y.numpy()
    assert np.abs(dx.sum(1, dtype=np.float64)).max() <= 2e-5
    sl = slice(0, 256)
    y64, g64 = yh[sl].astype(np.float64), g[sl].astype(np.float64)
    want = y64 * (g64 - (g64 * y64).sum(1, keepdims=True))
    assert np.abs(dx[sl] - want).max() <= 2e-6 * np.abs(want).max() + 1e-9
    gy = cref.binary("mul", g[sl], yh[sl])                         # the four-kernel form of ops.Softmax.backward
    ref = cref.binary("sub", gy, cref.binary("mul", yh[sl], cref.reduce("sum", gy, 1)[:, None]))
    assert np.abs(dx[sl] - ref).max() <= 1e-5 * np.abs(ref).max()


MASKED_CASES = [((2, 4, 128, 128), (128, 128)), ((8, 12, 1024, 1024), (1024, 1024)), ((3, 5, 100, 100), (100, 100)),
                ((2, 3, 7, 7), (7, 7)), ((1, 4, 1, 128), (1, 1, 1, 128)), ((6, 130), (6, 130)), ((5, 33), (33,))]


@pytest.mark.parametrize("xs,ms", MASKED_CASES)
def test_fused_masked_softmax_is_the_three_op_chain(xs, ms, monkeypatch):
    """`(x * scale).masked_fill(mask, -inf).softmax(last)` as one kernel, and its backward as one
    kernel: values and input gradients bit-identical to the chain of kernels they replace
    (same arithmetic in the same order), masked probabilities exactly 0 with gradient +0,
    every row summing to 1; a slice is also held against float64 (2e-6)."""
    require_gpu()
    from dlgrad_amd import ops
    rng = np.random.default_rng(60)
    x = rng.standard_normal(xs, dtype=np.float32) * 3
    g = rng.standard_normal(xs, dtype=np.float32)
    mask = (rng.random(ms) < 0.4).astype(np.float32)
    mask.reshape(-1, ms[-1])[:, 0] = 0                      # no row is masked entirely
    scale, dim = 0.125 * 1.37, len(xs) - 1

    def run(fused):
        monkeypatch.setattr(ops, "use_fused_masked_softmax", (lambda *a: False) if not fused else ops.use_fused_masked_softmax)
        t = Tensor(x, device="hip", requires_grad=True)
        y = t.masked_softmax(Tensor(mask, device="hip"), scale, dim=dim)
        node = type(y._ctx).__name__
        (y * Tensor(g, device="hip")).sum().backward()
        return y, t.grad, node

    (y1, g1, n1), (y0, g0, n0) = run(True), run(False)
    assert n1 == "MaskedSoftmax" and n0 != "MaskedSoftmax"
    if hip.COMPILE_ONLY:
        return
    y1, g1, y0, g0 = y1.numpy(), g1.numpy(), y0.numpy(), g0.numpy()
    np.testing.assert_array_equal(y1.view(np.uint32), y0.view(np.uint32))
    np.testing.assert_array_equal(g1.view(np.uint32), g0.view(np.uint32))
    full = np.broadcast_to(mask.reshape((1,) * (len(xs) - mask.ndim) + mask.shape), xs) > 0
    assert not y1[full].any() and not g1[full].any() and not np.signbit(g1[full]).any()
    assert np.abs(y1.sum(-1, dtype=np.float64) - 1).max() <= 1e-5
    sl = (slice(0, 1),) * (len(xs) - 2) + (slice(0, 64),)
    z = np.where(full[sl], -np.inf, x[sl].astype(np.float64) * np.float32(scale))
    e = np.exp(z - z.max(-1, keepdims=True))
    want = e / e.sum(-1, keepdims=True)
    assert np.abs(y1[sl] - want).max() <= 2e-6
    gw = want * (g[sl] - (g[sl] * want).sum(-1, keepdims=True)) * scale
    assert np.abs(g1[sl] - gw).max() <= 2e-6 * max(1.0, np.abs(gw).max())


@pytest.mark.parametrize("shape", [(2, 3, 64, 64), (1, 2, 1024, 1024), (3, 128, 128), (2, 100, 100), (8, 12, 1024, 1024)])
def test_the_kept_causal_mask_is_computed_instead_of_read(shape):
    """The (T, T) causal mask that ops.causal_mask builds once and keeps is recognised by its allocation: the scaled
    masked softmax and its backward then form "column > row" from the indices instead of reading a mask row per
    score row.  Same kernels otherwise: the results must have the bits of a run with an equal mask that lives
    in another buffer (and is therefore read)."""
    require_gpu()
    from dlgrad_amd import ops
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    T = shape[-1]
    rng = np.random.default_rng(75)
    big = int(np.prod(shape)) > 1 << 24
    x = rng.standard_normal(shape, dtype=np.float32)
    g = rng.standard_normal(shape, dtype=np.float32)
    kept = ops.causal_mask(T, Device.HIP)
    other = Buffer.from_numpy(np.triu(np.ones((T, T), np.float32), 1), Device.HIP)
    xb, gb = Buffer.from_numpy(x, Device.HIP), Buffer.from_numpy(g, Device.HIP)
    seen = set(hip.requested_kernels)
    y1 = xb.masked_softmax(kept, 0.125)
    d1 = y1.masked_softmax_bwd(gb, kept, 0.125)
    new = {(n, p) for n, p in hip.requested_kernels - seen if "softmax" in n} if not seen >= hip.requested_kernels else set()
    y0 = xb.masked_softmax(other, 0.125)
    d0 = y0.masked_softmax_bwd(gb, other, 0.125)
    assert hip.HIP._is_causal_mask(kept, T, T) and not hip.HIP._is_causal_mask(other, T, T)
    assert all(p[-1] in ("causal", True) for _, p in new)
    if hip.COMPILE_ONLY:
        return
    if not big:
        np.testing.assert_array_equal(kept.numpy(), other.numpy())
    for name, a, b in (("y", y1, y0), ("dx", d1, d0)):
        a, b = a.numpy(), b.numpy()
        assert (a.view(np.uint32) == b.view(np.uint32)).all(), name
        if name == "y":
            assert not np.triu(a.reshape(-1, T, T)[0], 1).any()


def test_masked_softmax_falls_back_to_the_chain_where_the_kernel_does_not_fit():
    """Rows too long for registers, a mask that does not line up with the trailing dims, or
    another axis: the op-by-op chain runs, with the same result as on the CPU oracle (1e-6)."""
    require_gpu()
    from dlgrad_amd import ops
    rng = np.random.default_rng(61)
    for xs, ms, dim in (((2, 70000), (70000,), 1), ((4, 6, 8), (4, 1, 8), 2), ((4, 8), (4, 8), 0)):
        x = rng.standard_normal(xs, dtype=np.float32)
        mask = (rng.random(ms) < 0.3).astype(np.float32)
        mask[..., 0] = 0
        if dim == 0:
            mask[0] = 0
        t, m = Tensor(x, device="hip"), Tensor(mask, device="hip")
        assert not ops.use_fused_masked_softmax(t, m, dim)
        got = t.masked_softmax(m, 0.5, dim=dim).numpy()
        want = Tensor(x).masked_softmax(Tensor(mask), 0.5, dim=dim).numpy()
        check(got, want, 1e-6, f"masked softmax chain {xs} {ms} dim {dim}")


@pytest.mark.parametrize("shape", [(2, 4, 128, 32), (1, 12, 1024, 64), (3, 2, 100, 20), (2, 1, 257, 64), (5, 64, 16)])
def test_causal_attention_node_equals_the_op_by_op_chain(shape, monkeypatch):
    """nn.causal_attention on the hip device runs the chain's own kernels with the causal structure
    known (k read in place, score tiles above the diagonal skipped, products cut at the diagonal):
    output and the gradients of q, k and v must be bit-identical to
    (q @ k^T).masked_softmax(mask, scale) @ v, and close to a float64 evaluation (1e-5)."""
    require_gpu()
    from dlgrad_amd import nn, ops
    rng = np.random.default_rng(70)
    q, k, v, g = (rng.standard_normal(shape, dtype=np.float32) for _ in range(4))
    scale = shape[-1] ** -0.5

    def run(fused):
        monkeypatch.setattr(ops, "use_fused_causal_attention", (lambda *a: False) if not fused else ops.use_fused_causal_attention)
        ts = [Tensor(a, device="hip", requires_grad=True) for a in (q, k, v)]
        y = nn.causal_attention(*ts, scale)
        node = type(y._ctx).__name__
        (y * Tensor(g, device="hip")).sum().backward()
        return node, [y.numpy()] + [t.grad.numpy() for t in ts]

    (n1, fused), (n0, chain) = run(True), run(False)
    assert n1 == "CausalAttention" and n0 != "CausalAttention"
    if hip.COMPILE_ONLY:
        return
    for name, a, b in zip(("y", "dq", "dk", "dv"), fused, chain):
        assert (a.view(np.uint32) == b.view(np.uint32)).all(), f"{name} {shape}"
    T = shape[-2]
    q64, k64, v64 = (a.astype(np.float64) for a in (q, k, v))
    s = np.where(np.triu(np.ones((T, T), bool), 1), -np.inf, (q64 @ np.swapaxes(k64, -1, -2)) * scale)
    e = np.exp(s - s.max(-1, keepdims=True))
    want = (e / e.sum(-1, keepdims=True)) @ v64
    assert np.abs(fused[0] - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("shape", [(2, 2, 256, 32), (2, 1, 257, 64), (1, 3, 130, 8)])
def test_causal_attention_never_reads_what_it_skipped(shape):
    """The score and dP tiles above the diagonal are left unwritten, so they hold whatever the
    pool's blocks held before.  With the pool's free blocks filled with NaN first, output and
    gradients must still be finite and bit-identical to a run on clean memory: nothing that
    was skipped may enter a sum, whether the rows take the 16-byte or the 4-byte kernels."""
    require_gpu()
    from dlgrad_amd import nn
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    rng = np.random.default_rng(71)
    q, k, v, g = (rng.standard_normal(shape, dtype=np.float32) for _ in range(4))

    def run():
        ts = [Tensor(a, device="hip", requires_grad=True) for a in (q, k, v)]
        y = nn.causal_attention(*ts, 0.25)
        assert type(y._ctx).__name__ == "CausalAttention"
        (y * Tensor(g, device="hip")).sum().backward()
        return [y.numpy()] + [t.grad.numpy() for t in ts]

    clean = run()
    T = shape[-2]
    n_scores = int(np.prod(shape[:-2])) * T * T
    poison = [Buffer.from_numpy(np.full(n, np.nan, np.float32), Device.HIP)
              for n in (n_scores, n_scores, n_scores, int(np.prod(shape)), int(np.prod(shape)))]
    hip.lib().sync()
    del poison                                               # back to the pool, NaN and all
    dirty = run()
    if hip.COMPILE_ONLY:
        return
    for name, a, b in zip(("y", "dq", "dk", "dv"), dirty, clean):
        assert np.isfinite(a).all(), name
        assert (a.view(np.uint32) == b.view(np.uint32)).all(), name


@pytest.mark.parametrize("B,T,h,d", [(2, 128, 4, 32), (1, 1024, 12, 64), (3, 100, 2, 20), (2, 257, 1, 64), (4, 16, 2, 6), (2, 130, 3, 7)])
def test_attention_on_the_projections_equals_split_attend_merge(B, T, h, d, monkeypatch):
    """nn.causal_self_attention takes q, k, v as (B, T, h*d) and reads every head where it lies
    (strided product kernels) instead of transposing to (B, h, T, d) and back.  Output and the
    gradients of the three projections are bit-identical to reshape -> transpose -> attention ->
    transpose -> reshape, including head sizes that force 4-byte accesses."""
    require_gpu()
    from dlgrad_amd import nn, ops
    monkeypatch.setattr(hip.HIP, "ATTENTION_FUSED", False)       # the one-launch kernels for short sequences add in another order,
    monkeypatch.setattr(hip.HIP, "ATTENTION_FLASH", False)       # and so do the streaming kernels for long ones
    rng = np.random.default_rng(72)
    C = h * d
    q, k, v, g = (rng.standard_normal((B, T, C), dtype=np.float32) for _ in range(4))
    scale = d ** -0.5

    def run(fused):
        monkeypatch.setattr(ops, "use_fused_attention_heads", (lambda *a: False) if not fused else ops.use_fused_attention_heads)
        ts = [Tensor(a, device="hip", requires_grad=True) for a in (q, k, v)]
        y = nn.causal_self_attention(*ts, h, scale)
        node = type(y._ctx).__name__
        (y * Tensor(g, device="hip")).sum().backward()
        return node, [y.numpy()] + [t.grad.numpy() for t in ts]

    (n1, fused), (n0, chain) = run(True), run(False)
    assert n1 == "CausalAttentionHeads" and n0 != "CausalAttentionHeads"
    if hip.COMPILE_ONLY:
        return
    for name, a, b in zip(("y", "dq", "dk", "dv"), fused, chain):
        assert a.shape == (B, T, C)
        assert (a.view(np.uint32) == b.view(np.uint32)).all(), f"{name} B{B} T{T} h{h} d{d}"


def attention_float64(q, k, v, g, h, scale):
    """Causal attention on (B, T, h*d) projections and its gradients for upstream g, in float64."""
    B, T, C = q.shape
    d = C // h
    q, k, v, g = (a.astype(np.float64).reshape(B, T, h, d).transpose(0, 2, 1, 3) for a in (q, k, v, g))
    s = np.where(np.triu(np.ones((T, T), bool), 1), -np.inf, (q @ k.transpose(0, 1, 3, 2)) * scale)
    e = np.exp(s - s.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    y = p @ v
    dv = p.transpose(0, 1, 3, 2) @ g
    dp = g @ v.transpose(0, 1, 3, 2)
    ds = p * (dp - (dp * p).sum(-1, keepdims=True)) * scale
    dq, dk = ds @ k, ds.transpose(0, 1, 3, 2) @ q
    return [a.transpose(0, 2, 1, 3).reshape(B, T, C) for a in (y, dq, dk, dv)]


@pytest.mark.parametrize("B,T,h,d", [(2, 128, 4, 32), (64, 128, 4, 32), (3, 100, 2, 20), (1, 1, 1, 4), (2, 33, 3, 8), (5, 65, 2, 28),
                                     (2, 31, 8, 4)])
@pytest.mark.parametrize("stacked", [False, True])
def test_short_attention_in_one_launch_per_pass(B, T, h, d, stacked, monkeypatch):
    """Up to 128 positions and head widths up to 32 (multiples of 4): one block per (sequence, head)
    holds q, k, v and the scores in LDS, so attention is one launch forward and one backward,
    from separate (B, T, C) projections or from one interleaved (B, T, 3C) projection.  The dot
    products add in another order than the chain of launches does, so the check is against
    float64: 2e-6 of the largest entry for the context and each gradient; the probabilities
    above the diagonal are exact zeros and nothing unwritten is read (free memory full of NaN)."""
    require_gpu()
    from dlgrad_amd import nn, ops
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    rng = np.random.default_rng(74)
    C = h * d
    q, k, v, g = (rng.standard_normal((B, T, C), dtype=np.float32) for _ in range(4))
    scale = d ** -0.5
    want = None if hip.COMPILE_ONLY else attention_float64(q, k, v, g, h, scale)
    poison = [Buffer.from_numpy(np.full(n, np.nan, np.float32), Device.HIP) for n in (B * h * T * T, 3 * B * T * C, B * T * C)]
    hip.lib().sync()
    del poison

    def run():
        if stacked:
            qkv = Buffer.from_numpy(np.ascontiguousarray(np.concatenate([q, k, v], axis=2)), Device.HIP)
            before = hip.launch_count
            y, p = qkv.causal_attention_qkv(h, scale)
            dg = qkv.causal_attention_qkv_bwd(p, Buffer.from_numpy(g, Device.HIP), h, scale, y)
            launches = hip.launch_count - before
            if hip.COMPILE_ONLY:
                return launches, None, None
            dg = dg.numpy()
            return launches, [y.numpy(), dg[:, :, :C], dg[:, :, C:2 * C], dg[:, :, 2 * C:]], p.numpy()
        bufs = [Buffer.from_numpy(a, Device.HIP) for a in (q, k, v, g)]
        before = hip.launch_count
        y, p = bufs[0].causal_attention(bufs[1], bufs[2], h, scale)
        grads = bufs[0].causal_attention_bwd(bufs[1], bufs[2], p, bufs[3], h, scale, y)
        launches = hip.launch_count - before
        if hip.COMPILE_ONLY:
            return launches, None, None
        return launches, [y.numpy()] + [a.numpy() for a in grads], p.numpy()

    launches, got, p = run()
    assert launches == 2, launches
    monkeypatch.setattr(hip.HIP, "ATTENTION_FUSED", False)
    chain_launches, chain, _ = run()
    assert chain_launches > 2
    if hip.COMPILE_ONLY:
        return
    assert p.shape == (B, h, T, T) and not np.triu(p, 1).any() and np.isfinite(p).all()
    assert np.abs(p.sum(-1, dtype=np.float64) - 1).max() <= 1e-5
    for name, a, w, c in zip(("y", "dq", "dk", "dv"), got, want, chain):
        assert np.isfinite(a).all(), name
        bound = 2e-6 * max(1.0, np.abs(w).max())
        assert np.abs(a - w).max() <= bound, f"{name}: {np.abs(a - w).max():.3g} > {bound:.3g}"
        assert np.abs(c - w).max() <= bound, f"chain {name}"


@pytest.mark.parametrize("B,T,h,d", [(1, 1024, 12, 64), (2, 257, 1, 64), (3, 100, 2, 20), (2, 384, 3, 48), (1, 130, 2, 32), (2, 129, 5, 4),
                                     (1, 640, 2, 64), (1, 1, 2, 64), (1, 777, 1, 36)])
@pytest.mark.parametrize("stacked", [False, True])
def test_streaming_attention_against_float64(B, T, h, d, stacked, monkeypatch):
    """Sequences beyond the one-launch kernels (or heads wider than 32): keys and values stream past
    128 queries per block with an online softmax, and the backward pass recomputes the probabilities
    from the kept log-sum-exp per row -- no T x T tensor is kept, the forward is one launch, the backward a
    row-sum launch, the key-side launch that also writes dS, and the product dQ = dS K.  Context and all
    three gradients against float64 at 2e-6 of the largest entry, for ragged T and head widths that are
    padded on the chip, from separate (B, T, C) projections and from one interleaved (B, T, 3C) one, with
    free memory full of NaN (nothing unwritten is read); the kept statistics against float64 too.  The chain
    of products and softmax launches over stored T x T tensors (DLGRAD_HIP_ATTENTION_FLASH=0) meets the
    same bound; the two add in different orders, so their bits are not compared."""
    require_gpu()
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    monkeypatch.setattr(hip.HIP, "ATTENTION_FUSED", False)               # (shapes the one-launch kernels would take go to the streaming ones)
    rng = np.random.default_rng(75 + T)
    C = h * d
    q, k, v, g = (rng.standard_normal((B, T, C), dtype=np.float32) for _ in range(4))
    scale = d ** -0.5
    want = None if hip.COMPILE_ONLY else attention_float64(q, k, v, g, h, scale)
    poison = [Buffer.from_numpy(np.full(n, np.nan, np.float32), Device.HIP) for n in (B * h * T * T, 3 * B * T * C, B * T * C, B * h * T)]
    hip.lib().sync()
    del poison

    def run():
        if stacked:
            qkv = Buffer.from_numpy(np.ascontiguousarray(np.concatenate([q, k, v], axis=2)), Device.HIP)
            before = hip.launch_count
            y, p = qkv.causal_attention_qkv(h, scale)
            dg = qkv.causal_attention_qkv_bwd(p, Buffer.from_numpy(g, Device.HIP), h, scale, y)
            launches = hip.launch_count - before
            if hip.COMPILE_ONLY:
                return launches, None, None
            dg = dg.numpy()
            return launches, [y.numpy(), dg[:, :, :C], dg[:, :, C:2 * C], dg[:, :, 2 * C:]], p.numpy()
        bufs = [Buffer.from_numpy(a, Device.HIP) for a in (q, k, v, g)]
        before = hip.launch_count
        y, p = bufs[0].causal_attention(bufs[1], bufs[2], h, scale)
        grads = bufs[0].causal_attention_bwd(bufs[1], bufs[2], p, bufs[3], h, scale, y)
        launches = hip.launch_count - before
        if hip.COMPILE_ONLY:
            return launches, None, None
        return launches, [y.numpy()] + [a.numpy() for a in grads], p.numpy()

    launches, got, lse = run()
    assert launches == 4, launches
    monkeypatch.setattr(hip.HIP, "ATTENTION_FLASH", False)
    chain_launches, chain, p = run()
    assert chain_launches > 4
    if hip.COMPILE_ONLY:
        return
    assert lse.size == B * h * T and (lse.shape == (B, h, T) or T == 1) and p.shape == (B, h, T, T)    # (for T = 1 the two shapes hold as many numbers)
    lse = lse.reshape(B, h, T)
    s64 = np.einsum("bthd,bshd->bhts", q.reshape(B, T, h, d).astype(np.float64), k.reshape(B, T, h, d).astype(np.float64)) * scale
    s64 = np.where(np.tril(np.ones((T, T), bool)), s64, -np.inf)
    want_lse = np.log(np.exp(s64 - s64.max(-1, keepdims=True)).sum(-1)) + s64.max(-1)
    assert np.abs(lse - want_lse).max() <= 2e-6 * max(1.0, np.abs(want_lse).max())
    for name, a, w, c in zip(("y", "dq", "dk", "dv"), got, want, chain):
        assert np.isfinite(a).all(), name
        bound = 2e-6 * max(1.0, np.abs(w).max())
        assert np.abs(a - w).max() <= bound, f"{name}: {np.abs(a - w).max():.3g} > {bound:.3g}"
        assert np.abs(c - w).max() <= bound, f"chain {name}"


def test_short_attention_leaves_other_shapes_to_the_chain_of_launches():
    """Longer sequences, wider heads, head widths that are no multiple of 4 and operands that do not
    sit on 16-byte boundaries do not fit the LDS tiles or the 16-byte loads of the one-block kernels."""
    from dlgrad_amd.runtime.hip import HIP
    fits = HIP._attention_fits
    assert fits(128, 32, 256, (0, 16, 4096), (96,))
    assert not fits(129, 32, 256, (0,), (96,)) and not fits(128, 36, 256, (0,), (108,)) and not fits(64, 6, 8, (0,), (12,))
    assert not fits(64, 8, 8, (4,), (24,)) and not fits(64, 8, 8, (0,), (25,)) and not fits(64, 8, 0, (0,), (24,))


@pytest.mark.parametrize("B,T,h,d", [(2, 128, 4, 32), (1, 1024, 12, 64), (3, 100, 2, 20), (2, 33, 3, 7)])
def test_stacked_qkv_attention_equals_three_projections_and_attention(B, T, h, d, monkeypatch):
    """nn.self_attention_qkv with weights that nn.stack_parameters placed back to back: one
    projection, heads read out of its (B, T, 3C) result.  The context and the three weight
    gradients have the bits of the separate route (three projections, attention on the
    projections); dx adds its 3C terms in one accumulator instead of three partial sums and
    agrees to 1e-5 of the largest entry (a 2304-term fp32 sum at C = 768)."""
    require_gpu()
    from dlgrad_amd import nn, ops
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_SPLITK", False)     # bit-equality is between products that add k in one piece (a plain product of few tiles may be given a tile that cuts k)
    rng = np.random.default_rng(73)
    C = h * d
    x, g = (rng.standard_normal((B, T, C), dtype=np.float32) for _ in range(2))
    ws = [rng.standard_normal((C, C), dtype=np.float32) * C ** -0.5 for _ in range(3)]
    scale = d ** -0.5

    def run(fused):
        monkeypatch.setattr(ops, "use_fused_qkv_attention", (lambda *a: False) if not fused else ops.use_fused_qkv_attention)
        xt = Tensor(x, device="hip", requires_grad=True)
        wt = [Tensor(w, device="hip", requires_grad=True) for w in ws]
        nn.stack_parameters(wt)
        assert ops.stacked(*wt) or hip.COMPILE_ONLY
        for t, w in zip(wt, ws):
            check(t.numpy(), w, 0, "stacking keeps the values")
        y = nn.self_attention_qkv(xt, *wt, h, scale)
        node = type(y._ctx).__name__
        (y * Tensor(g, device="hip")).sum().backward()
        return node, [y.numpy(), xt.grad.numpy()] + [t.grad.numpy() for t in wt]

    (n1, fused), (n0, chain) = run(True), run(False)
    assert n1 == "SelfAttentionQKV" and n0 != "SelfAttentionQKV"
    if hip.COMPILE_ONLY:
        return
    for name, a, b in zip(("y", "dx", "dwq", "dwk", "dwv"), fused, chain):
        if name == "dx":
            assert np.abs(a - b).max() <= 1e-5 * np.abs(b).max(), name
        else:
            assert (a.view(np.uint32) == b.view(np.uint32)).all(), f"{name} B{B} T{T} h{h} d{d}"


@pytest.mark.parametrize("B,T,C,H", [(2, 64, 48, 192), (1, 100, 36, 50), (4, 256, 384, 1536)])
def test_feed_forward_with_fused_epilogues_equals_the_four_ops(B, T, C, H, monkeypatch):
    """nn.mlp_relu and nn.Linear(x, residual): the ReLU, its gradient select and the residual
    addition ride on the stores of the products.  Output and every gradient (input, both weights,
    residual) have the bits of linear -> relu -> linear -> add run op by op."""
    require_gpu()
    from dlgrad_amd import nn, ops
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_SPLITK", False)     # bit-equality is with the unsplit products (an epilogue is never split; a plain product of few tiles may be)
    rng = np.random.default_rng(B * T + C)
    x, r, g = (rng.standard_normal((B, T, C), dtype=np.float32) for _ in range(3))
    w1 = rng.standard_normal((H, C), dtype=np.float32) * C ** -0.5
    w2 = rng.standard_normal((C, H), dtype=np.float32) * H ** -0.5
    usable = ops.use_fused_epilogues

    def run(fused, what):
        monkeypatch.setattr(ops, "use_fused_epilogues", usable if fused else (lambda *a: False))
        ts = [Tensor(a, device="hip", requires_grad=True) for a in (x, w1, w2, r)]
        if what == "mlp":
            y = nn.mlp_relu(*ts)
        elif what == "mlp_plain":
            y = nn.mlp_relu(*ts[:3])
        else:
            lin = nn.Linear(H, C, bias=False)
            lin.weight = ts[2]
            h = Tensor(np.abs(np.resize(x, (B, T, H))), device="hip", requires_grad=True)
            ts[0] = h
            y = lin(h, ts[3])
        node = type(y._ctx).__name__
        (y * Tensor(g, device="hip")).sum().backward()
        return node, [y.numpy()] + [t.grad.numpy() for t in ts if t.grad is not None]

    for what, node in (("mlp", "MLPRelu"), ("mlp_plain", "MLPRelu"), ("linear", "LinearNTAdd")):
        (n1, fused), (n0, chain) = run(True, what), run(False, what)
        assert n1 == node and n0 != node, (what, n1, n0)
        assert len(fused) == len(chain) == (4 if what == "mlp_plain" else 5 if what == "mlp" else 4)
        if hip.COMPILE_ONLY:
            continue
        for i, (a, b) in enumerate(zip(fused, chain)):
            assert a.shape == b.shape and (a.view(np.uint32) == b.view(np.uint32)).all(), f"{what} output/gradient {i}"


@pytest.mark.parametrize("B,h,d,rows,n,masked", [(1, 4, 32, 128, 128, True), (1, 4, 32, 128, 37, False), (3, 2, 64, 300, 300, True),
                                                 (2, 3, 20, 70, 65, False), (2, 12, 64, 1024, 1000, True), (1, 1, 7, 5, 1, False)])
def test_attention_for_one_new_position_in_one_launch(B, h, d, rows, n, masked, monkeypatch):
    """nn.cached_attention on the hip device: scores, softmax and context of the decoding branch
    (examples/gpt.py:58-63) by one kernel, checked against float64 numpy and against the three-launch
    form it replaces, both to 2e-6 of the largest entry (the dot products are added in another order)."""
    require_gpu()
    from dlgrad_amd.runtime.hip import HIP
    rng = np.random.default_rng(B * 100 + n)
    C = h * d
    q = rng.standard_normal((B, 1, C), dtype=np.float32)
    ks, vs = (rng.standard_normal((rows, B, C), dtype=np.float32) for _ in range(2))
    hidden = (rng.random((1, n)) < 0.3).astype(np.float32) if masked else None
    if masked:
        hidden[0, 0] = 0.0                                         # something is always visible
    scale = d ** -0.5
    qd, kd, vd = dev(q), dev(ks), dev(vs)
    hd = dev(hidden) if masked else None

    def run(fused):
        monkeypatch.setattr(HIP, "DECODE_FUSED", fused)
        before = hip.launch_count
        y = qd.cached_attention(kd, vd, n, h, scale, hd)
        return hip.launch_count - before, y.numpy()

    (l1, got), (l0, chain) = run(True), run(False)
    assert l1 == 1 and l0 >= 3, (l1, l0)
    q64 = q.astype(np.float64).reshape(B, h, d)
    k64 = ks[:n].astype(np.float64).reshape(n, B, h, d)
    v64 = vs[:n].astype(np.float64).reshape(n, B, h, d)
    s = np.einsum("bhd,nbhd->bhn", q64, k64) * scale
    if masked:
        s = np.where(hidden[0] > 0, -np.inf, s)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("bhn,nbhd->bhd", p, v64).reshape(B, 1, C)
    if hip.COMPILE_ONLY:
        return
    top = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-6 * top, "one-launch attention vs float64"
    assert np.abs(got - chain).max() <= 2e-6 * top, "one-launch attention vs product-softmax-product"


def test_cached_attention_checks_its_stores_on_the_host():
    require_gpu()
    q = dev(np.zeros((2, 1, 8), np.float32))
    store = dev(np.zeros((5, 2, 8), np.float32))
    with pytest.raises(ValueError):
        q.cached_attention(store, store, 6, 2, 1.0)                       # more positions than rows
    with pytest.raises(ValueError):
        q.cached_attention(dev(np.zeros((5, 1, 8), np.float32)), store, 3, 2, 1.0)   # another batch size
    with pytest.raises(ValueError):
        dev(np.zeros((2, 2, 8), np.float32)).cached_attention(store, store, 3, 2, 1.0)   # two positions
    assert q.cached_attention(store, store, 5, 2, 1.0).shape == (2, 1, 8)
