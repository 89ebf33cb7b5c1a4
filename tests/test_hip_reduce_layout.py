"""GPU parity: reductions, arg-max, permutations, embedding, cross-entropy helpers and
the fused row softmax against the C oracle.

Tolerances (task statement): reductions 1e-5 relative -- judged on |hip - f64| not being
worse than that, or on hip being at least as close to float64 as the CPU path is, because
a -ffast-math fp32 sum over millions of values is itself ~1e-5..1e-4 away from the true sum;
max, arg-max, permutes, gathers and the CE helpers are bit-exact."""
import numpy as np
import pytest

from dlgrad_amd.buffer import Buffer
from dlgrad_amd.device import Device
from dlgrad_amd.helpers import CustomOps
from oracle import cref
from tests.hip_util import check, dev, rel_err, require_gpu
from dlgrad_amd.runtime import hip

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(5)


def f32(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


def check_sum_like(got, x64_result, cpu_result, what):
    """1e-5 relative to the scale of the result, or at least as close to float64 as the CPU path."""
    if hip.COMPILE_ONLY:
        return
    got = np.asarray(got, np.float64)
    scale = np.maximum(np.abs(x64_result), np.abs(x64_result).mean() if np.ndim(x64_result) else 0) + 1e-30
    e_hip = np.max(np.abs(got - x64_result) / scale)
    e_cpu = np.max(np.abs(np.asarray(cpu_result, np.float64) - x64_result) / scale)
    assert got.shape == np.shape(x64_result), what
    assert e_hip <= 1e-5 or e_hip <= e_cpu, f"{what}: hip err {e_hip:.2e}, cpu err {e_cpu:.2e}"


SHAPES = [(5,), (4, 7), (3, 4, 5), (2, 3, 4, 5), (64, 1000), (1000, 64), (1024, 1024), (16, 4, 128, 128),
          (16, 128, 128), (4097, 3), (3, 4099), (2048, 65), (70000, 2), (2, 300000)]


@pytest.mark.parametrize("shape", SHAPES)
def test_sum_mean_max_every_axis(shape):
    require_gpu()
    x = f32(*shape)
    x64 = x.astype(np.float64)
    b = dev(x)
    check_sum_like(b.sum().numpy(), x64.sum(), cref.reduce("sum", x), f"sum all {shape}")
    check_sum_like(b.mean().numpy(), x64.mean(), cref.reduce("mean", x), f"mean all {shape}")
    check(b.max().numpy(), cref.reduce("max", x), 0, f"max all {shape}")
    for d in range(len(shape)):
        for keep in (False, True):
            want_shape = tuple(1 if i == d else s for i, s in enumerate(shape)) if keep else \
                tuple(s for i, s in enumerate(shape) if i != d)
            check_sum_like(b.sum(d, keepdim=keep).numpy(), x64.sum(d).reshape(want_shape),
                           cref.reduce("sum", x, d).reshape(want_shape), f"sum {shape} axis {d}")
        check_sum_like(b.mean(d).numpy(), x64.mean(d), cref.reduce("mean", x, d), f"mean {shape} axis {d}")
        check(b.max(d).numpy(), cref.reduce("max", x, d), 0, f"max {shape} axis {d}")


@pytest.mark.parametrize("shape", [(4096, 4096), (16384, 8192)])
def test_reductions_at_bench_sizes(shape):
    require_gpu()
    x = f32(*shape)
    b = dev(x)
    x64 = x.astype(np.float64)
    check_sum_like(b.sum().numpy(), x64.sum(), cref.reduce("sum", x), "sum all")
    check(b.max().numpy(), x.max(), 0, "max all")
    for d in (0, 1):
        check_sum_like(b.sum(d).numpy(), x64.sum(d), cref.reduce("sum", x, d), f"sum axis {d}")
        check(b.max(d).numpy(), x.max(d), 0, f"max axis {d}")


def test_max_of_minus_inf_rows_matches_reference_start_value():
    require_gpu()
    x = np.full((5, 130), -np.inf, np.float32)
    x[2, 7] = 3.0
    check(dev(x).max(1).numpy(), cref.reduce("max", x, 1), 0, "max rows -inf")
    check(dev(x).max(0).numpy(), cref.reduce("max", x, 0), 0, "max cols -inf")
    check(dev(x[:2]).max().numpy(), cref.reduce("max", x[:2]), 0, "max all -inf")


@pytest.mark.parametrize("shape", [(128, 10), (10000, 10), (1, 65), (1, 50304), (7, 1000), (300, 257), (5, 50304), (3, 5003),
                                   (5000, 300), (70000, 33), (9, 2048), (257, 32)])
def test_argmax_bit_exact_with_ties(shape):
    require_gpu()
    x = RNG.integers(0, 5, shape).astype(np.float32)         # few distinct values: many ties
    for d in (0, 1):
        want = cref.argmax(x, d).reshape((1, shape[1]) if d == 0 else (shape[0], 1))
        check(dev(x).argmax(d).numpy(), want, 0, f"argmax {shape} dim {d}")
    y = f32(*shape)
    check(dev(y).argmax(1).numpy(), y.argmax(1).astype(np.float32).reshape(-1, 1), 0, "argmax random")


@pytest.mark.parametrize("form", ["direct", "staged"])
@pytest.mark.parametrize("L", [1, 2, 7, 8, 9, 10, 16, 17, 31, 32])
def test_argmax_of_many_short_rows(L, form, monkeypatch):
    """Row counts above 4096 with L <= 32: a thread per row with 8-byte loads where the length is
    even and the rows are 8-byte aligned ("direct"), else -- and wherever "staged" is chosen -- through
    LDS, 256 rows a block; the last block is ragged (row counts that are no multiple of 256, of 4,
    and an odd total) and a view that starts 4 bytes into its block takes the narrow loads."""
    require_gpu()
    monkeypatch.setattr(hip, "ARGMAX_SHORT_ROWS", form)
    for R in (4096, 4099, 10001):
        x = RNG.integers(0, 4, (R, L)).astype(np.float32)
        want = cref.argmax(x, 1).reshape(R, 1)
        check(dev(x).argmax(1).numpy(), want, 0, f"argmax ({R}, {L})")
        flat = np.concatenate([np.zeros(1, np.float32), x.reshape(-1)])
        view = Buffer(Buffer.from_numpy(flat, Device.HIP).ptr + 1, x.shape, Device.HIP)
        check(view.argmax(1).numpy(), want, 0, f"argmax ({R}, {L}) misaligned")


def test_argmax_never_selects_minus_inf():
    """The scan starts at (-FLT_MAX, index 0) and moves on `v > best` only (cpu_kernel.py:497-499):
    rows of -inf answer 0; every kernel variant must agree.  (NaN is left out: the reference
    compiles that comparison under -ffinite-math-only, which leaves its outcome to the compiler.)"""
    require_gpu()
    for shape in ((6, 10), (6, 300), (6, 4096), (600, 70), (5000, 10)):
        x = np.full(shape, -np.inf, np.float32)
        x[1, shape[1] - 1] = -1e30
        x[2, 5] = 7.0
        x[4, 2] = x[4, shape[1] - 2] = 9.0
        for d in (0, 1):
            want = cref.argmax(x, d).reshape((1, shape[1]) if d == 0 else (shape[0], 1))
            check(dev(x).argmax(d).numpy(), want, 0, f"argmax {shape} dim {d} with -inf")


PERMS = [((256, 512), (1, 0)), ((8, 12, 64, 128), (0, 1, 3, 2)), ((4, 128, 8, 64), (0, 2, 3, 1)), ((132, 260), (1, 0)),
         ((2048, 768), (1, 0)), ((4, 7), (1, 0)), ((64, 784), (1, 0)), ((10, 64), (1, 0)), ((128, 128), (1, 0)), ((512, 128), (1, 0)),
         ((2, 3, 4), (0, 2, 1)), ((2, 3, 4), (2, 0, 1)), ((2, 3, 4), (1, 0, 2)), ((2, 3, 4, 5), (0, 2, 1, 3)),
         ((2, 3, 4, 5), (0, 1, 3, 2)), ((2, 3, 4, 5), (3, 2, 1, 0)), ((2, 3, 4, 5), (1, 3, 0, 2)),
         ((16, 128, 4, 32), (0, 2, 1, 3)), ((16, 4, 128, 32), (0, 1, 3, 2)), ((16, 4, 128, 32), (0, 2, 1, 3)),
         ((1000, 333), (1, 0)), ((3, 1, 5), (2, 1, 0)), ((5,), (0,)), ((2, 3, 4, 6), (0, 1, 2, 3)),
         # row pitches that are multiples of 2 KiB: diagonal tile order, 64- and 128-wide tiles, ragged last tiles
         ((1028, 512), (1, 0)), ((3, 1028, 512), (0, 2, 1)), ((1024, 1536), (1, 0)), ((4100, 4096), (1, 0)),
         ((3, 1156, 4608), (0, 2, 1))]


@pytest.mark.parametrize("shape,order", PERMS)
def test_permute_bit_exact(shape, order):
    require_gpu()
    x = f32(*shape)
    check(dev(x).permute(order).numpy(), cref.permute(x, order), 0, f"permute {shape} {order}")


def test_transpose_at_bench_size_is_exact_and_its_own_inverse():
    require_gpu()
    x = f32(8192, 4096)
    t = dev(x).transpose(0, 1)
    check(t.numpy(), x.T, 0, "8192 x 4096 transpose")
    check(t.transpose(0, 1).numpy(), x, 0, "transposed twice")


def test_transpose_helpers():
    require_gpu()
    x = f32(6, 9)
    check(dev(x).T.numpy(), x.T, 0, "T")
    x4 = f32(2, 3, 4, 5)
    check(dev(x4).transpose(1, 2).numpy(), x4.transpose(0, 2, 1, 3), 0, "transpose(1,2)")
    # the op the reference's other runtimes register under UnaryOps.TRANSPOSE, with their keywords
    from dlgrad_amd.dispatch import dispatcher
    from dlgrad_amd.helpers import UnaryOps
    got = dispatcher.dispatch(UnaryOps.TRANSPOSE, Device.HIP, x=dev(x4), out_stride=(60, 5, 15, 1), out_shape=(2, 4, 3, 5), dim0=1, dim1=2)
    check(Buffer(got, (2, 4, 3, 5), Device.HIP).numpy(), x4.transpose(0, 2, 1, 3), 0, "UnaryOps.TRANSPOSE")


@pytest.mark.parametrize("V,W,idx_shape", [(100, 32, (4, 16)), (65, 128, (16, 128)), (128, 128, (128,)),
                                          (50, 7, (33,)), (1000, 768, (64,))])
def test_embedding_gather_bit_exact_and_scatter_add(V, W, idx_shape):
    require_gpu()
    table = f32(V, W)
    idx = RNG.integers(0, V, idx_shape).astype(np.float32)
    check(dev(table).embedding(dev(idx)).numpy(), cref.embedding(table, idx), 0, "gather")
    g = f32(*idx_shape, W)
    got = dev(table).embedding(dev(idx), backward=True, upstream_grad=dev(g)).numpy()
    want = cref.embedding_backward((V, W), idx, g)
    if hip.COMPILE_ONLY:
        return
    if idx.size <= 512:
        # one segment: rows are added in index order starting from zero, as the reference's loop does
        np.testing.assert_array_equal(got, want)
    else:
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_embedding_scatter_add_is_deterministic_and_atomics_path_agrees(monkeypatch):
    require_gpu()
    V, W, n = 300, 96, 5000
    idx = np.minimum(RNG.zipf(1.3, n) - 1, V - 1).astype(np.float32)
    g, t = f32(n, W), dev(f32(V, W))
    runs = [t.embedding(dev(idx), backward=True, upstream_grad=dev(g)).numpy() for _ in range(3)]
    monkeypatch.setattr(hip, "EMB_ORDERED", False)
    atomic = t.embedding(dev(idx), backward=True, upstream_grad=dev(g)).numpy()
    if hip.COMPILE_ONLY:
        return
    np.testing.assert_array_equal(runs[0], runs[1])
    np.testing.assert_array_equal(runs[0], runs[2])
    want = np.zeros((V, W))
    np.add.at(want, idx.astype(int), g.astype(np.float64))
    np.testing.assert_allclose(runs[0], want, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(atomic, want, rtol=1e-4, atol=1e-4)


def ordered_scatter_model(V, idx, g, segment=512):
    """The summation order of the ordered scatter-add, in float32: inside a segment of 512
    positions an id's rows are added in index order starting from 0; an id that occurs in
    several segments then adds those partial sums in segment order, starting from the first."""
    out = np.zeros((V, g.shape[-1]), np.float32)
    ids = idx.reshape(-1).astype(np.int64)
    rows = g.reshape(ids.size, -1)
    partials = {}
    for s0 in range(0, ids.size, segment):
        acc = {}
        for j in range(s0, min(ids.size, s0 + segment)):
            acc[ids[j]] = acc.get(ids[j], np.zeros(rows.shape[1], np.float32)) + rows[j]
        for k, v in acc.items():
            partials.setdefault(k, []).append(v)
    for k, parts in partials.items():
        total = parts[0]
        for v in parts[1:]:
            total = total + v
        out[k] = total
    return out


def scatter_order_model(V, W, idx, g):
    """What the deterministic scatter-add must give, bit for bit: the sequential order of the reference's loop where
    the one-launch form for small tables applies, the segment-wise order of the three-launch form elsewhere."""
    n = int(np.asarray(idx).size)
    return ordered_scatter_model(V, idx, g, segment=n if hip.HIP.scatter_small_fits(V, W, n) else 512)


@pytest.mark.parametrize("small", [False, True])
@pytest.mark.parametrize("W", [4, 7, 96, 2052])
@pytest.mark.parametrize("pattern", ["same", "pairs", "span", "zipf", "hot"])
def test_ordered_scatter_add_has_exactly_the_documented_summation_order(pattern, W, small, monkeypatch):
    """Bit-exact against a float32 model of the order, for id patterns that exercise one id
    filling whole segments (its 512 wavefronts split the columns, most get none), adjacent
    pairs, ids that occur once in every segment (merge only), Zipf ids, and one hot id among
    unique ones; W = 7 takes the 4-byte kernels, W = 2052 needs two passes over a row.  Table
    rows no index names come out as zeros although nothing zero-fills the table first.
    small: the one-launch form for small tables (strictly the reference's sequential order); otherwise
    the three-launch form, forced also where the one-launch form would apply."""
    require_gpu()
    V, n = 3000, 1536 + 77
    if small and not hip.HIP.scatter_small_fits(V, W, n):
        pytest.skip("too many wavefronts for the one-launch form")
    if not small:
        monkeypatch.setattr(hip.HIP, "scatter_small_fits", staticmethod(lambda V, W, n: False))
    rng = np.random.default_rng(W)
    ids = {"same": np.full(n, 5), "pairs": np.repeat(rng.permutation(V)[:(n + 1) // 2], 2)[:n],
           "span": np.tile(rng.permutation(V)[:512], 4)[:n], "zipf": np.minimum(rng.zipf(1.1, n) - 1, V - 1),
           "hot": np.where(np.arange(n) % 11 == 0, 7, rng.permutation(V)[:n])}[pattern].astype(np.float32)
    g = rng.standard_normal((n, W), dtype=np.float32)
    g[3] = -0.0                                                   # 0 + (-0) is +0, as in the reference's `+=`
    poison = np.full((V, W), np.nan, np.float32)                  # whatever the output block held before must not show
    keep = [dev(poison) for _ in range(3)]
    del keep
    n0 = hip.launch_count
    got = dev(f32(V, W)).embedding(dev(ids), backward=True, upstream_grad=dev(g)).numpy()
    assert hip.launch_count - n0 == (1 if small else 3)
    if not hip.COMPILE_ONLY:
        want = scatter_order_model(V, W, ids, g)
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
        if small:                                                 # the reference's loop, literally
            np.testing.assert_array_equal(got.view(np.uint32), cref.embedding_backward((V, W), ids, g).view(np.uint32))


@pytest.mark.parametrize("V,W,n", [(40, 2, 2000), (1, 1, 300), (70000, 4, 5), (130, 8, 32768), (64, 12, 40000)])
def test_scatter_add_on_narrow_tall_and_long_inputs(V, W, n):
    """Two columns shared by many wavefronts, a one-element table, a table far taller than the index
    list (zero blocks dominate), the longest list the ordered kernel takes, and one beyond it (atomics)."""
    require_gpu()
    idx = RNG.integers(0, V, n).astype(np.float32)
    g = f32(n, W)
    got = dev(f32(V, W)).embedding(dev(idx), backward=True, upstream_grad=dev(g)).numpy()
    if hip.COMPILE_ONLY:
        return
    if n <= 32768:
        want = scatter_order_model(V, W, idx, g)
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    want = np.zeros((V, W))
    np.add.at(want, idx.astype(int), g.astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)


def test_embedding_scatter_with_heavy_collisions():
    require_gpu()
    V, W, n = 50, 64, 4096
    idx = np.minimum(RNG.zipf(1.1, n) - 1, V - 1).astype(np.float32)    # most ids are 0..3
    g = f32(n, W)
    got = dev(f32(V, W)).embedding(dev(idx), backward=True, upstream_grad=dev(g)).numpy()
    want = np.zeros((V, W))
    np.add.at(want, idx.astype(int), g.astype(np.float64))
    if not hip.COMPILE_ONLY:
        np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)


def test_cross_entropy_helpers_bit_exact():
    require_gpu()
    lsm = f32(2048, 65)
    t = RNG.integers(0, 65, (2048, 1)).astype(np.float32)
    check(Buffer.ce_forward(dev(lsm), dev(t)).numpy(), cref.ce_forward(lsm, t).reshape(1, -1), 0, "ce_forward")
    p = dev(lsm)
    Buffer.ce_backward(op=CustomOps.CE_BACKWARD, device=p.device, x=p, target=dev(t))
    want = lsm.copy()
    cref.ce_backward_(want, t)
    check(p.numpy(), want, 0, "ce_backward in place")


@pytest.mark.parametrize("shape", [(8, 10), (16, 4, 128, 128), (2048, 65), (96, 1024), (4, 50304), (5, 4099), (3, 2052)])
def test_fused_softmax_matches_the_five_kernel_composition(shape):
    require_gpu()
    x = f32(*shape) * 3
    m = cref.reduce("max", x, len(shape) - 1)[..., None]
    e = cref.unary("exp", cref.binary("sub", x, m))
    s = cref.reduce("sum", e, len(shape) - 1)[..., None]
    check(dev(x).softmax(len(shape) - 1).numpy(), cref.binary("div", e, s), 2e-6, f"softmax {shape}")
    lsm = cref.binary("sub", cref.binary("sub", x, m), cref.unary("log", s))
    got = dev(x).log_softmax(len(shape) - 1).numpy()
    if not hip.COMPILE_ONLY:
        np.testing.assert_allclose(got, lsm, rtol=2e-6, atol=2e-6)


def test_softmax_with_causal_minus_inf_mask_gives_exact_zeros():
    require_gpu()
    att = f32(2, 4, 128, 128)
    mask = 1 - np.tril(np.ones((128, 128), np.float32))
    filled = Buffer.masked_fill(dev(att), dev(mask), float("-inf"))
    p = filled.softmax(3).numpy()
    if not hip.COMPILE_ONLY:
        assert np.all(p[..., np.triu_indices(128, 1)[0], np.triu_indices(128, 1)[1]] == 0)
        np.testing.assert_allclose(p.sum(-1), 1.0, rtol=1e-5)


@pytest.mark.parametrize("W", [1, 64, 384, 1000])
def test_row_store_writes_the_row_the_device_index_names(W):
    """dst[(int)idx, :] = src with idx read on the device (the cache append of a captured decoding
    step), alone and for two destinations in one launch; an index outside the rows writes nothing.
    Bit-exact."""
    require_gpu()
    rng = np.random.default_rng(W)
    R = 9
    a0, b0 = (rng.standard_normal((R, 2, W), dtype=np.float32) for _ in range(2))
    ra, rb = (rng.standard_normal((1, 2 * W), dtype=np.float32) for _ in range(2))
    for row in (0, 4, 8, 9, -1):
        a, b, idx = dev(a0), dev(b0), dev(np.array([[row]], np.float32))
        before = hip.launch_count
        a.row_store_(dev(ra), idx, also=(b, dev(rb)))
        launches = hip.launch_count - before
        wa, wb = a0.copy(), b0.copy()
        if 0 <= row < R:
            wa[row], wb[row] = ra.reshape(2, W), rb.reshape(2, W)
        check(a.numpy(), wa, 0, f"first destination, row {row}")
        check(b.numpy(), wb, 0, f"second destination, row {row}")
        assert launches == 1
        c = dev(a0)
        c.row_store_(dev(rb), idx)
        wc = a0.copy()
        if 0 <= row < R:
            wc[row] = rb.reshape(2, W)
        check(c.numpy(), wc, 0, f"single destination, row {row}")
    with pytest.raises(ValueError):
        dev(a0).row_store_(dev(ra), dev(np.zeros((1, 1), np.float32)), also=(dev(np.zeros((R, 3, W), np.float32)), dev(rb)))


def _ce_float64(logits, t):
    """(sum of the row losses, mean-scaled gradient) in float64 (ops.py:337-370: forward sums, backward divides by N)."""
    z = logits.astype(np.float64)
    z = z - z.max(1, keepdims=True)
    lsm = z - np.log(np.exp(z).sum(1, keepdims=True))
    n = logits.shape[0]
    grad = np.exp(lsm)
    grad[np.arange(n), t] -= 1.0
    return -lsm[np.arange(n), t].sum(), grad / n


@pytest.mark.parametrize("N,V", [(1, 65), (1, 64), (1, 50304), (2, 65), (4, 64), (300, 1000), (3, 50304)])
@pytest.mark.parametrize("fused", [True, False])
def test_cross_entropy_loss_and_gradient_single_rows_included(N, V, fused, monkeypatch):
    """A single row collapses to a flat index space in the launcher, where the one-hot column must
    still be found; targets 0, V-1 and in between."""
    require_gpu()
    from dlgrad_amd import Tensor, ops
    monkeypatch.setattr(ops, "FUSED", fused)
    logits = f32(N, V) * 2
    for t0 in (0, V - 1, V // 3):
        t = (np.arange(N) * 7 + t0) % V
        a = Tensor(logits, requires_grad=True, device="hip")
        loss = a.cross_entropy_loss(Tensor(t.astype(np.float32).reshape(N, 1), device="hip"))
        loss.backward()
        got_loss, got_grad = float(loss.numpy()), a.grad.numpy()
        if hip.COMPILE_ONLY:
            continue
        want_loss, want_grad = _ce_float64(logits, t)
        assert abs(got_loss - want_loss) <= 1e-5 * abs(want_loss), (N, V, t0)
        assert np.abs(got_grad - want_grad).max() <= 1e-5 * np.abs(want_grad).max(), (N, V, t0)
        assert (got_grad[np.arange(N), t] < 0).all() and (np.delete(got_grad[0], t[0]) > 0).all()


@pytest.mark.parametrize("N,V", [(1, 64), (1, 65), (2048, 65), (64, 50304), (33, 4100), (7, 2048), (5, 100003), (9, 1028), (3, 44)])
def test_ce_row_statistics_stand_in_for_the_stored_log_softmax(N, V):
    """The forward keeps (max, log-sum) per row instead of the (N, V) log-softmax.  The max is exact; the
    sum is added in one pass with a running maximum, so log-sum, picked log-probs and the gradient rebuilt
    from the logits agree with the stored-tensor route to rounding (1e-6 of the largest entry), and with
    float64 to the tolerance of the element-wise ops."""
    require_gpu()
    logits = f32(N, V) * 3
    logits[0, :min(V, 40)] = -np.inf                                # exp gives exact zeros; the row still has finite entries
    t = RNG.integers(0, V, (N, 1)).astype(np.float32)
    t[0] = V - 1
    x, dt = dev(logits), dev(t)
    lsm, picked_old = x.log_softmax_gather(dt)
    m, ls, picked = x.ce_stats(dt)
    check(m.numpy().ravel(), cref.reduce("max", logits, 1), 0, "row max")
    if hip.COMPILE_ONLY:
        return
    z = logits.astype(np.float64)
    ls64 = np.log(np.exp(z - z.max(1, keepdims=True)).sum(1))
    assert np.abs(ls.numpy().ravel() - ls64).max() <= 2e-6 * max(1.0, np.abs(ls64).max())
    assert np.abs(picked.numpy() - picked_old.numpy()).max() <= 2e-6 * np.abs(picked_old.numpy()).max()
    one = Buffer.from_scalar(1.0)
    for up in (one, dev(np.float32(0.37).reshape(1, 1))):
        new, old = x.ce_grad_logits(m, ls, dt, up, float(N)).numpy(), lsm.ce_grad(dt, up, float(N)).numpy()
        assert np.abs(new - old).max() <= 2e-6 * np.abs(old).max()
        assert (new[0, :min(V, 40)] == 0).all()
        # rows of whole 16-byte items take a kernel with a block per (row, run of columns): the same operations
        # in the same order as the element-wise launch, so the same bits
        rows_kernel = hip.HIP.CE_GRAD_ROWS
        hip.HIP.CE_GRAD_ROWS = False
        try:
            flat = x.ce_grad_logits(m, ls, dt, up, float(N)).numpy()
        finally:
            hip.HIP.CE_GRAD_ROWS = rows_kernel
        np.testing.assert_array_equal(new.view(np.uint32), flat.view(np.uint32))


def test_indices_outside_their_table_touch_nothing():
    """Token ids and class targets are data: one that is negative or too large must not read or
    write outside its tensor.  Gather gives a row of zeros, scatter-add skips the row, the
    cross-entropy helpers pick 0 and subtract nothing; every in-range entry is unaffected."""
    require_gpu()
    V, W, n = 50, 64, 700                                          # two segments of the ordered scatter-add
    table, g = f32(V, W), f32(n, W)
    idx = RNG.integers(0, V, n).astype(np.float32)
    bad = np.array([3, 100, 511, 512, 650])
    idx[bad] = [-1.0, float(V), 1e9, -7.0, float(V + 3)]
    ok = np.ones(n, bool)
    ok[bad] = False
    got = dev(table).embedding(dev(idx)).numpy()
    if not hip.COMPILE_ONLY:
        np.testing.assert_array_equal(got[ok], table[idx[ok].astype(int)])
        assert not got[bad].any()
    want = cref.embedding_backward((V, W), idx[ok], g[ok])
    for ordered in (True, False):
        old = hip.EMB_ORDERED
        hip.EMB_ORDERED = ordered
        try:
            got = dev(table).embedding(dev(idx), backward=True, upstream_grad=dev(g)).numpy()
        finally:
            hip.EMB_ORDERED = old
        if not hip.COMPILE_ONLY:
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5, err_msg=f"ordered={ordered}")
    lsm = f32(6, 10)
    t = np.array([0, 9, -1, 10, 3, 1e6], np.float32).reshape(6, 1)
    inside = np.array([True, True, False, False, True, False])
    picked = Buffer.ce_forward(dev(lsm), dev(t)).numpy().ravel()
    p = dev(lsm)
    Buffer.ce_backward(op=CustomOps.CE_BACKWARD, device=p.device, x=p, target=dev(t))
    after = p.numpy()
    _, _, picked2 = dev(lsm).ce_stats(dev(t))
    _, picked3 = dev(lsm).log_softmax_gather(dev(t))
    if not hip.COMPILE_ONLY:
        want_pick = np.where(inside, lsm[np.arange(6), np.where(inside, t.ravel(), 0).astype(int)], 0)
        np.testing.assert_array_equal(picked, want_pick)
        want_after = lsm.copy()
        want_after[np.arange(6)[inside], t.ravel()[inside].astype(int)] -= 1
        np.testing.assert_array_equal(after, want_after)
        assert not picked2.numpy().ravel()[~inside].any() and not picked3.numpy().ravel()[~inside].any()


def test_tensors_without_elements_and_with_one():
    """Extents of 0 and 1 in every op family: no launch of an empty grid, the shapes the oracle gives, and for
    the reductions what an empty loop leaves behind (0 for a sum, -FLT_MAX for a max, 0 / 0 for a mean)."""
    require_gpu()
    e, one = np.zeros((0, 4), np.float32), np.full((1, 1), 3.0, np.float32)
    for a, b in ((e, e), (one, one), (np.zeros((3, 0), np.float32), np.zeros((3, 0), np.float32))):
        check((dev(a) + dev(b)).numpy(), cref.binary("add", a, b), 0, f"add {a.shape}")
        check(dev(a).exp().numpy(), cref.unary("exp", a), 1e-6, f"exp {a.shape}")
        check(dev(a).permute((1, 0)).numpy(), cref.permute(a, (1, 0)), 0, f"transpose {a.shape}")
        for dim in (0, 1):
            for op in ("sum", "max"):
                check(getattr(dev(a), op)(dim).numpy(), cref.reduce(op, a, dim), 0, f"{op} {a.shape} over {dim}")
    for op in ("sum", "max"):
        check(getattr(dev(e), op)(-1).numpy(), cref.reduce(op, e), 0, f"{op} of nothing")
        check(getattr(dev(one), op)(-1).numpy(), cref.reduce(op, one), 0, f"{op} of one element")
    if not hip.COMPILE_ONLY:
        assert np.isnan(dev(e).mean(-1).numpy())
    check(dev(e).matmul(dev(np.ones((4, 3), np.float32))).numpy(), np.zeros((0, 3), np.float32), 0, "no rows times a matrix")
    check(dev(np.ones((2, 0), np.float32)).matmul(dev(np.ones((0, 3), np.float32))).numpy(), np.zeros((2, 3), np.float32), 0, "empty k")
    check(dev(one).matmul(dev(one)).numpy(), np.full((1, 1), 9.0, np.float32), 0, "1 x 1")
    check(dev(e).softmax(1).numpy(), e, 0, "softmax of no rows")
    check(dev(e).argmax(1).numpy(), np.zeros((0, 1), np.float32), 0, "argmax of no rows")
