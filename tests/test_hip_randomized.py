"""GPU parity on seeded random shapes: the launcher's classification of an op (vectorised
row/column/scalar broadcast, strided fallback, 16-byte or 4-byte accesses, tile and block
choices) depends on shape, strides and alignment, so the shape space is sampled rather than
listed.  Every case is compared with the C oracle or a float64 closed form at the bars of the
fixed-shape tests: bit-exact for + - * selects comparisons permutes max argmax, 1e-6 for
division and transcendental maps, 1e-5 for sums (or at least as close to float64 as the CPU
path), 1e-4 for matmul.  Inputs include zero-sized dims, size-1 dims in every position,
extents that are no multiple of 4, and views that start at odd offsets."""
import numpy as np
import pytest

from dlgrad_amd.buffer import Buffer
from dlgrad_amd.device import Device
from dlgrad_amd.runtime import hip
from oracle import cref
from tests.hip_util import check, dev, require_gpu

pytestmark = pytest.mark.gpu
DIMS = [1, 1, 2, 3, 4, 5, 7, 8, 12, 16, 31, 33, 64, 100]


def shape_of(rng, rank, big=False):
    return tuple(int(rng.choice(DIMS if not big else DIMS + [128, 257])) for _ in range(rank))


def misaligned(a):
    """The same values as a device view that starts 4 bytes into its block."""
    flat = np.concatenate([np.zeros(1, np.float32), a.reshape(-1)])
    base = Buffer.from_numpy(flat, Device.HIP)
    return Buffer(base.ptr + 1, a.shape, Device.HIP)


@pytest.mark.parametrize("seed", range(12))
def test_random_broadcast_binary_ops(seed):
    require_gpu()
    rng = np.random.default_rng(1000 + seed)
    for _ in range(12):
        rank = int(rng.integers(1, 5))
        xs = shape_of(rng, rank, big=rank <= 2)
        ys = tuple(1 if rng.random() < 0.4 else d for d in xs)
        if rng.random() < 0.25:
            ys = ys[int(rng.integers(0, rank)):] or (1,)              # lower-rank right operand
        x = rng.standard_normal(xs, dtype=np.float32)
        y = (rng.standard_normal(ys, dtype=np.float32) + np.float32(3.0)) * np.float32(rng.choice([-1, 1]))
        xd = misaligned(x) if rng.random() < 0.3 else dev(x)
        yd = misaligned(y) if rng.random() < 0.3 else dev(y)
        for op, tol in (("add", 0), ("sub", 0), ("mul", 0), ("div", 1e-6)):
            got = getattr(xd, f"__{op if op != 'div' else 'truediv'}__")(yd).numpy()
            check(got, cref.binary(op, x, y), tol, f"{op} {xs} {ys}")
        check((xd > yd).numpy(), (x > np.broadcast_to(y, xs)).astype(np.float32), 0, f"gt {xs} {ys}")


@pytest.mark.parametrize("seed", range(6))
def test_random_unary_select_and_fill_ops(seed):
    require_gpu()
    rng = np.random.default_rng(2000 + seed)
    for _ in range(10):
        xs = shape_of(rng, int(rng.integers(1, 5)), big=True)
        x = rng.standard_normal(xs, dtype=np.float32)
        xd = misaligned(x) if rng.random() < 0.3 else dev(x)
        check(xd.exp().numpy(), cref.unary("exp", x), 1e-6, f"exp {xs}")
        check((-xd).numpy(), -x, 0, f"neg {xs}")
        check((xd ** 2).numpy(), x * x, 0, f"pow2 {xs}")
        check(xd.relu().numpy(), np.where(x > 0, x, np.float32(0)), 0, f"relu {xs}")
        check(xd.clamp(-1, 1).numpy(), cref.clamp(x, -1, 1), 0, f"clamp {xs}")
        pos = np.abs(x) + np.float32(1e-3)
        check(dev(pos).log().numpy(), cref.unary("log", pos), 1e-6, f"log {xs}")
        check(dev(pos).sqrt().numpy(), np.sqrt(pos), 1e-6, f"sqrt {xs}")
        ms = tuple(1 if rng.random() < 0.5 else d for d in xs)
        mask = (rng.random(ms) < 0.5).astype(np.float32)
        check(Buffer.masked_fill(xd, dev(mask), -np.inf).numpy(), cref.masked_fill(x, mask, -np.inf), 0, f"masked_fill {xs} {ms}")
        other = rng.standard_normal(xs, dtype=np.float32)
        check(dev(np.broadcast_to(mask, xs).copy()).where(xd, dev(other)).numpy(),
              np.where(np.broadcast_to(mask, xs) > 0, x, other), 0, f"where {xs}")


@pytest.mark.parametrize("seed", range(8))
def test_random_reductions_argmax_and_permutes(seed):
    require_gpu()
    rng = np.random.default_rng(3000 + seed)
    for _ in range(10):
        rank = int(rng.integers(1, 5))
        xs = shape_of(rng, rank, big=rank <= 2)
        x = rng.standard_normal(xs, dtype=np.float32)
        xd = misaligned(x) if rng.random() < 0.3 else dev(x)
        x64 = x.astype(np.float64)
        for d in [-1] + list(range(rank)):
            want = x64.sum() if d == -1 else x64.sum(d)
            got = xd.sum(d).numpy().reshape(np.shape(want))
            if not hip.COMPILE_ONLY:
                ref = cref.reduce("sum", x, d).reshape(np.shape(want)).astype(np.float64)
                scale = np.abs(x64).sum() if d == -1 else np.abs(x64).sum(d)
                err_gpu, err_cpu = np.abs(got - want), np.abs(ref - want)
                assert (err_gpu <= 1e-5 * np.abs(want) + 1e-7 * scale).all() or (err_gpu <= err_cpu + 1e-12).all(), \
                    f"sum {xs} dim {d}"
            check(xd.max(d).numpy().reshape(np.shape(want)), x.max() if d == -1 else x.max(d), 0, f"max {xs} dim {d}")
        order = tuple(int(v) for v in rng.permutation(rank))
        check(xd.permute(order).numpy(), np.transpose(x, order), 0, f"permute {xs} {order}")
        if rank == 2:
            t = rng.integers(0, 4, xs).astype(np.float32)                # ties everywhere
            for d in (0, 1):
                want = cref.argmax(t, d).reshape((1, xs[1]) if d == 0 else (xs[0], 1))
                check(dev(t).argmax(d).numpy(), want, 0, f"argmax {xs} dim {d}")


@pytest.mark.parametrize("seed", range(6))
def test_random_matmuls_plain_and_transposed(seed):
    require_gpu()
    rng = np.random.default_rng(4000 + seed)
    for _ in range(8):
        M, Kd, N = (int(rng.choice([1, 3, 4, 7, 16, 33, 64, 100, 130])) for _ in range(3))
        batch = tuple(int(rng.choice([1, 2, 3])) for _ in range(int(rng.integers(0, 3))))
        yb = tuple(1 if rng.random() < 0.4 else b for b in batch)
        x = rng.standard_normal(batch + (M, Kd), dtype=np.float32)
        y = rng.standard_normal(yb + (Kd, N), dtype=np.float32) * np.float32(Kd ** -0.5)
        want = x.astype(np.float64) @ y.astype(np.float64)
        xd, yd = dev(x), dev(y)
        scale = float(np.abs(want).max()) + 1e-30
        nn_ = xd.matmul(yd).numpy()
        if not hip.COMPILE_ONLY:
            assert np.abs(nn_ - want).max() <= 1e-4 * scale, f"matmul {x.shape} {y.shape}"
        yt = np.ascontiguousarray(np.swapaxes(y, -1, -2))
        xt = np.ascontiguousarray(np.swapaxes(x, -1, -2))
        nt = xd.matmul_nt(dev(yt)).numpy()
        if x.size == Kd and not hip.COMPILE_ONLY:           # a single row: one wavefront per output splits the k sum over its lanes
            assert np.abs(nt - nn_).max() <= 2e-6 * scale, f"NT {x.shape} {yt.shape}"
        else:
            check(nt, nn_, 0, f"NT {x.shape} {yt.shape}")                                 # same bits as the plain product
        check(dev(xt).matmul_tn(yd).numpy(), nn_, 0, f"TN {xt.shape} {y.shape}")


def test_zero_sized_tensors_go_through_every_op_family():
    require_gpu()
    z = dev(np.zeros((0, 5), np.float32))
    assert (z + z).numpy().shape == (0, 5) and z.exp().numpy().shape == (0, 5)
    assert z.permute((1, 0)).numpy().shape == (5, 0)
    assert z.sum(0).numpy().shape == (5,) and not z.sum(0).numpy().any()
    w = dev(np.ones((5, 3), np.float32))
    assert z.matmul(w).numpy().shape == (0, 3)
    e = dev(np.ones((4, 0), np.float32)).matmul(dev(np.ones((0, 6), np.float32))).numpy()     # empty inner dim: zeros
    assert e.shape == (4, 6) and not e.any()


@pytest.mark.parametrize("seed", range(6))
def test_random_embedding_gathers_and_ordered_scatter_adds(seed):
    """Random table sizes, row widths (4-byte and 16-byte kernels), index counts on either side of
    the 512-position segment size and id distributions from all-distinct to one id everywhere:
    the gather is bit-exact, the scatter-add bit-exact against the float32 model of its summation
    order (index order inside segments of 512 positions, then the segment sums in order)."""
    require_gpu()
    from tests.test_hip_reduce_layout import scatter_order_model
    rng = np.random.default_rng(5000 + seed)
    for _ in range(6):
        V = int(rng.choice([1, 3, 50, 700, 5000]))
        W = int(rng.choice([1, 4, 6, 32, 100, 260]))
        n = int(rng.choice([1, 5, 511, 512, 513, 1300, 2100]))
        kind = rng.choice(["uniform", "zipf", "same", "few"])
        ids = {"uniform": rng.integers(0, V, n), "zipf": np.minimum(rng.zipf(1.2, n) - 1, V - 1),
               "same": np.full(n, V - 1), "few": rng.integers(0, min(V, 3), n)}[kind].astype(np.float32)
        table = rng.standard_normal((V, W), dtype=np.float32)
        g = rng.standard_normal((n, W), dtype=np.float32)
        t = dev(table)
        check(t.embedding(dev(ids)).numpy(), table[ids.astype(np.int64)], 0, f"gather V{V} W{W} n{n} {kind}")
        got = t.embedding(dev(ids), backward=True, upstream_grad=dev(g)).numpy()
        if hip.COMPILE_ONLY:
            continue
        want = scatter_order_model(V, W, ids, g)
        assert (got.view(np.uint32) == want.view(np.uint32)).all(), f"scatter V{V} W{W} n{n} {kind}"


@pytest.mark.parametrize("seed", range(4))
def test_random_masked_softmax_equals_its_chain(seed):
    """Random ranks, row lengths (16-byte and 4-byte kernels, one wavefront or a block per row),
    mask shapes that cover one row, the trailing two dims or the whole tensor, and scales: the
    fused forward and backward kernels give the bits of the mul / masked_fill / softmax chain."""
    require_gpu()
    from dlgrad_amd import Tensor, ops
    rng = np.random.default_rng(6000 + seed)
    for _ in range(6):
        rank = int(rng.integers(2, 5))
        L = int(rng.choice([1, 3, 8, 33, 64, 100, 256, 1000, 4096]))     # up to what the one-wavefront backward holds
        lead = tuple(int(rng.choice([1, 2, 3, 5])) for _ in range(rank - 1))
        xs = lead + (L,)
        keep = int(rng.integers(1, rank + 1))                      # the mask spans the last `keep` dims
        ms = xs[rank - keep:]
        x = rng.standard_normal(xs, dtype=np.float32) * 4
        g = rng.standard_normal(xs, dtype=np.float32)
        mask = (rng.random(ms) < 0.5).astype(np.float32)
        mask.reshape(-1, L)[:, int(rng.integers(0, L))] = 0       # every row keeps an entry
        scale = float(rng.choice([1.0, 0.125, 0.3]))
        outs = []
        for fused in (True, False):
            t, m = Tensor(x, device="hip", requires_grad=True), Tensor(mask, device="hip")
            if fused:
                assert ops.use_fused_masked_softmax(t, m, rank - 1), (xs, ms)
                y = t.masked_softmax(m, scale, dim=rank - 1)
            else:
                y = (t * scale).masked_fill(m, float("-inf")).softmax(dim=rank - 1)
            (y * Tensor(g, device="hip")).sum().backward()
            outs.append((y.numpy(), t.grad.numpy()))
        if hip.COMPILE_ONLY:
            continue
        assert (outs[0][0].view(np.uint32) == outs[1][0].view(np.uint32)).all(), f"forward {xs} {ms} {scale}"
        assert (outs[0][1].view(np.uint32) == outs[1][1].view(np.uint32)).all(), f"backward {xs} {ms} {scale}"


@pytest.mark.parametrize("seed", range(6))
def test_random_fused_launches_against_closed_forms(seed):
    """The launches that fold several ops into one, on random shapes, against numpy closed forms with the same
    roundings: token + position embedding (a gather, a gather, one fp32 add: bit-exact, ids outside their table
    read as zeros, any row width and alignment); the bias a product adds as it stores (the product's own bits
    plus one fp32 add); the end of a decoding step (first maximum; the token buffer's bound); the in-place SGD
    for many parameters per launch (two or four roundings per element)."""
    require_gpu()
    from dlgrad_amd import Tensor, nn
    rng = np.random.default_rng(7000 + seed)
    for _ in range(4):
        # ---- embedding sum
        V, P = int(rng.choice([1, 7, 65, 300])), int(rng.choice([1, 9, 40]))
        C = int(rng.choice([1, 3, 4, 6, 32, 100, 128]))
        B, T = int(rng.choice([1, 2, 5])), int(rng.choice([1, 4, 9, 33]))
        wte, wpe = rng.standard_normal((V, C), dtype=np.float32), rng.standard_normal((P, C), dtype=np.float32)
        ids = rng.integers(-1, V + 1, (B, T)).astype(np.float32)
        pos = rng.integers(-1, P + 1, (T,)).astype(np.float32)
        tt, pt = (misaligned(wte), misaligned(wpe)) if rng.random() < 0.5 else (dev(wte), dev(wpe))
        got = tt.embedding_sum(pt, dev(ids), dev(pos)).numpy()
        tok_rows = np.where(((ids >= 0) & (ids < V))[..., None], wte[np.clip(ids, 0, V - 1).astype(int)], np.float32(0))
        pos_rows = np.where(((pos >= 0) & (pos < P))[..., None], wpe[np.clip(pos, 0, P - 1).astype(int)], np.float32(0))
        check(got, (tok_rows + pos_rows[None]).astype(np.float32), 0, f"embedding sum V{V} P{P} C{C} B{B} T{T}")
        # ---- bias epilogue
        M, Kd, N = int(rng.choice([1, 2, 31, 130])), int(rng.choice([4, 12, 64, 100])), int(rng.choice([1, 3, 10, 64, 130]))
        x, w, b = rng.standard_normal((M, Kd), dtype=np.float32), rng.standard_normal((N, Kd), dtype=np.float32), rng.standard_normal((1, N), dtype=np.float32)
        xd, wd = dev(x), dev(w)
        plain = xd.matmul_nt(wd).numpy()
        check(xd.matmul_nt(wd, epi="bias", e=dev(b)).numpy(), plain + b, 0, f"bias {M}x{Kd}x{N}")
        # ---- the end of a decoding step
        Vn, rows = int(rng.choice([2, 65, 1000, 5000])), int(rng.choice([1, 3, 40]))
        logits = rng.standard_normal((1, Vn), dtype=np.float32)
        if rng.random() < 0.5:
            logits[0, rng.integers(0, Vn, 3)] = 9.0                  # ties: the first one wins
        s = float(rng.integers(-1, rows + 1))
        seq0 = rng.standard_normal((rows, 1), dtype=np.float32)
        tok, slot, seq = (Tensor(a, device="hip") for a in (np.array([[5.0]], np.float32), np.array([[s]], np.float32), seq0.copy()))
        assert nn.decode_append(Tensor(logits, device="hip"), tok, slot, seq)
        if not hip.COMPILE_ONLY:
            best = float(np.argmax(logits[0]))
            want_seq = seq0.copy()
            if 0 <= s + 1 < rows:
                want_seq[int(s) + 1, 0] = best
            assert tok.numpy()[0, 0] == best and slot.numpy()[0, 0] == s + 1, f"decode_next V{Vn} slot {s}"
            np.testing.assert_array_equal(seq.numpy(), want_seq)
        # ---- many parameters per SGD launch
        count, mu, lr = int(rng.choice([1, 5, 16, 17, 33])), float(rng.choice([0.0, 0.9])), np.float32(0.05)
        shapes = [(int(rng.integers(1, 700)),) for _ in range(count)]
        ps = [rng.standard_normal(sh, dtype=np.float32) for sh in shapes]
        gs = [rng.standard_normal(sh, dtype=np.float32) for sh in shapes]
        params = [Tensor(p.copy(), device="hip", requires_grad=True) for p in ps]
        opt = nn.optim.SGD(params, lr=float(lr), momentum=mu, graph_safe=True)
        vs = [np.zeros_like(p) for p in ps]
        for step in range(2):
            for p, g in zip(params, gs):
                p.grad = Tensor(g, device="hip")
            opt.step()
            for i, g in enumerate(gs):
                upd = g
                if mu:
                    vs[i] = (vs[i] * np.float32(mu)).astype(np.float32) + g
                    upd = vs[i]
                ps[i] = ps[i] - (upd * lr).astype(np.float32)
        for p, want in zip(params, ps):
            check(p.numpy(), want, 0, f"sgd x{count} mu={mu}")
