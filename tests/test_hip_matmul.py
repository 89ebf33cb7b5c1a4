"""GPU parity: fp32 MFMA matmul (2-D, batched, broadcast batches) against the C oracle's
i-k-j loops on small shapes and against BLAS/float64 on the large ones.

Bar (task statement): 1e-4 relative for fp32 matmul, measured as
max|got - want| / max|want| plus an element-wise check with atol = 1e-4 * max|want|.
Shape lists are the reference's (test/test_ops.py:77-103, :319-345; test/test_gpt.py:44-73)
plus the benchmark's sweep."""
import numpy as np
import pytest

from dlgrad_amd.runtime import hip
from oracle import cref
from tests.hip_util import check, dev, require_gpu

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(3)


def f32(*shape, scale=1.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


def check_mm(got, want, what):
    if hip.COMPILE_ONLY:
        return
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, f"{what}: {got.shape} vs {want.shape}"
    scale = np.abs(want).max() + 1e-30
    err = np.abs(got - want).max() / scale
    assert err <= 1e-4, f"{what}: {err:.3e}"


SHAPES_2D = [((2, 3), (3, 4)), ((1, 1), (1, 1)), ((5, 7), (7, 3)), ((128, 784), (784, 64)), ((128, 64), (64, 10)),
             ((33, 65), (65, 129)), ((64, 64), (64, 64)), ((128, 128), (128, 128)), ((100, 100), (100, 100)),
             ((257, 513), (513, 255)), ((2048, 128), (128, 128)), ((2048, 128), (128, 65)), ((4096, 4096), (4096, 1)),
             ((1, 4096), (4096, 4096)), ((300, 2), (2, 300))]


@pytest.mark.parametrize("xs,ys", SHAPES_2D)
def test_matmul_2d_vs_oracle(xs, ys):
    require_gpu()
    x, y = f32(*xs), f32(*ys, scale=xs[1] ** -0.5)
    want = cref.matmul(x, y) if xs[0] * xs[1] * ys[1] < 3e8 else x.astype(np.float64) @ y.astype(np.float64)
    check_mm((dev(x) @ dev(y)).numpy(), want, f"{xs}@{ys}")


def test_matmul_identity_and_transposed_operand_shapes():
    require_gpu()
    a = f32(200, 96)
    got = (dev(a) @ dev(np.eye(96, dtype=np.float32))).numpy()
    if not hip.COMPILE_ONLY:
        np.testing.assert_array_equal(got, a)            # exact: every product is a*1 or a*0
    g = f32(200, 40)
    # the backward shapes: A^T . G and G . B^T arrive as materialised transposes
    check_mm((dev(a).T @ dev(g)).numpy(), a.T.astype(np.float64) @ g, "A^T G")
    b = f32(96, 40)
    check_mm((dev(g) @ dev(b).T).numpy(), g.astype(np.float64) @ b.T, "G B^T")


SHAPES_ND = [((4, 5, 7), (4, 7, 3)), ((4, 5, 7), (1, 7, 3)), ((1, 5, 7), (4, 7, 3)), ((16, 128, 128), (1, 128, 128)),
             ((16, 128, 128), (1, 128, 512)), ((16, 128, 512), (1, 512, 128)), ((16, 128, 128), (1, 128, 65)),
             ((16, 128, 128), (16, 128, 64)), ((2, 3, 5, 7), (2, 3, 7, 4)), ((2, 1, 5, 7), (2, 3, 7, 4)),
             ((2, 3, 5, 7), (1, 1, 7, 4)), ((1, 3, 5, 7), (2, 1, 7, 4)), ((2, 3, 5, 7), (2, 1, 7, 4)),
             ((16, 4, 128, 32), (16, 4, 32, 128)), ((16, 4, 128, 128), (16, 4, 128, 32)),
             ((8, 23, 50, 100), (8, 23, 100, 10))]


@pytest.mark.parametrize("xs,ys", SHAPES_ND)
def test_matmul_batched_and_broadcast(xs, ys):
    require_gpu()
    x, y = f32(*xs), f32(*ys, scale=xs[-1] ** -0.5)
    got = dev(x).matmul(dev(y)).numpy()
    check_mm(got, cref.matmul(x, y), f"{xs}@{ys}")


def test_matmul_lower_rank_right_operand_is_padded():
    require_gpu()
    x, w = f32(16, 128, 128), f32(128, 64, scale=0.1)
    check_mm(dev(x).matmul(dev(w)).numpy(), x.astype(np.float64) @ w, "3d @ 2d")


@pytest.mark.parametrize("tile", list(__import__("dlgrad_amd.codegen.hip_kernel", fromlist=["x"]).MATMUL_CONFIGS))
@pytest.mark.parametrize("mnk", [(256, 256, 256), (130, 70, 50), (512, 384, 1000)])
def test_every_tile_configuration(tile, mnk, monkeypatch):
    require_gpu()
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
    M, N, Kd = mnk
    x, y = f32(M, Kd), f32(Kd, N, scale=Kd ** -0.5)
    check_mm((dev(x) @ dev(y)).numpy(), x.astype(np.float64) @ y, f"{tile} {mnk}")


@pytest.mark.parametrize("n", [1024, 2048, 4096])
def test_square_sweep_vs_float64_blas(n):
    require_gpu()
    x, y = f32(n, n), f32(n, n, scale=n ** -0.5)
    got = (dev(x) @ dev(y)).numpy()
    if n <= 2048:
        check_mm(got, x.astype(np.float64) @ y.astype(np.float64), f"{n}^3")
    elif not hip.COMPILE_ONLY:                                  # float64 on every 37th row: each tile row, all columns
        rows = np.arange(0, n, 37)
        want = x[rows].astype(np.float64) @ y.astype(np.float64)
        err = np.abs(got[rows] - want).max() / np.abs(want).max()
        assert err <= 1e-4, f"{n}^3: {err:.3e}"


def test_tall_skinny():
    require_gpu()
    x, y = f32(16384, 128), f32(128, 512, scale=128 ** -0.5)
    check_mm((dev(x) @ dev(y)).numpy(), x.astype(np.float64) @ y, "tall-skinny")


def test_every_tile_gives_the_same_bits(monkeypatch):
    """All tiles add the k terms of an output element in the same order, which is what lets
    the tile be chosen by timing without touching results."""
    require_gpu()
    from dlgrad_amd.codegen import hip_kernel as K
    from dlgrad_amd.runtime.hip import HIP
    x, y = f32(3, 200, 328), f32(3, 328, 196, scale=328 ** -0.5)
    xd, yd = dev(x), dev(y)
    outs = {}
    for tile in K.MATMUL_CONFIGS:
        monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
        outs[tile] = xd.matmul(yd).numpy()
    first = outs["64x64"]
    for tile, got in outs.items():
        check(got, first, 0, f"{tile} vs 64x64")


def test_whole_tile_form_gives_the_bits_of_the_guarded_form(monkeypatch):
    """A product cut into whole tiles runs the form of the kernel whose k loop carries no bounds tests: same loads, same
    products in the same order, so the same bits as the guarded form -- for every tile, with the operands as stored,
    transposed in place, and with a step on the accumulator as it is stored.  The shapes are two tiles by three with
    three or more k steps, so first, middle and last steps of the loop are all there."""
    require_gpu()
    from dlgrad_amd.codegen import hip_kernel as K
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_SPLITK", False)
    rng = np.random.default_rng(11)
    for tile, cfg in K.MATMUL_CONFIGS.items():
        bm, bn, _ = K.matmul_tile_shape(tile)
        M, N, Kd = 2 * bm, 3 * bn, max(3 * cfg[4], 192)
        x, y = rng.standard_normal((M, Kd), dtype=np.float32), rng.standard_normal((Kd, N), dtype=np.float32) * np.float32(Kd ** -0.5)
        e = rng.standard_normal((M, N), dtype=np.float32)
        xd, yd, ytd, xtd, ed = dev(x), dev(y), dev(np.ascontiguousarray(y.T)), dev(np.ascontiguousarray(x.T)), dev(e)
        monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
        runs = {"nn": lambda: xd.matmul(yd), "nt": lambda: xd.matmul_nt(ytd), "tn": lambda: xtd.matmul_tn(yd),
                "nn add": lambda: xd.matmul(yd, epi="add", e=ed), "nt relu": lambda: xd.matmul_nt(ytd, epi="relu"),
                "nn gate": lambda: xd.matmul(yd, epi="gate", e=ed)}
        for what, run in runs.items():
            monkeypatch.setattr(HIP, "MATMUL_EXACT", False)
            want = run().numpy()
            guarded = HIP.last_matmul_kernel
            monkeypatch.setattr(HIP, "MATMUL_EXACT", True)
            got = run().numpy()
            assert guarded and not guarded.endswith("_x") and HIP.last_matmul_kernel == guarded + "_x", (tile, what, guarded, HIP.last_matmul_kernel)
            check(got, want, 0, f"{tile} {what}: whole-tile form vs guarded form")
        check_mm(xd.matmul(yd).numpy(), x.astype(np.float64) @ y, f"{tile} whole-tile form")


def test_first_use_of_a_large_shape_times_the_tiles_and_remembers_the_winner(monkeypatch, tmp_path):
    require_gpu()
    from dlgrad_amd.runtime import hip as H
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_TUNED_FILE", str(tmp_path / "matmul_tuned.json"))
    monkeypatch.setattr(HIP, "MATMUL_FORCE", None)
    monkeypatch.setattr(HIP, "MATMUL_TUNE", True)
    monkeypatch.setattr(HIP, "_tuned", {})
    monkeypatch.setattr(HIP, "_tuned_new", {})
    M, Kd, N = 1000, 520, 776
    x, y = f32(M, Kd), f32(Kd, N, scale=Kd ** -0.5)
    n0 = H.launch_count
    got = (dev(x) @ dev(y)).numpy()
    assert H.launch_count == n0 + 1                     # the timing launches are not counted as work
    check_mm(got, x.astype(np.float64) @ y, "tuned shape")
    if H.COMPILE_ONLY:
        return
    key = f"1,{M},{N},{Kd},sk"                          # few tiles, k >= 512: timed with the split-k forms too, under a key of its own
    assert HIP._valid_tile(HIP._tuned[key]) and HIP._split_of(HIP._tuned[key])[0] in __import__("dlgrad_amd.codegen.hip_kernel", fromlist=["x"]).MATMUL_CONFIGS
    import json
    assert json.load(open(tmp_path / "matmul_tuned.json"))[key] == HIP._tuned[key]
    small = (dev(f32(64, 64)) @ dev(f32(64, 64))).numpy()         # below the threshold: the model picks, nothing is stored
    assert small.shape == (64, 64) and len(HIP._tuned) == 1


TRANSPOSED_CASES = [((64, 48), (40, 48)), ((130, 70), (50, 70)), ((200, 328), (196, 328)), ((97, 33), (45, 33)),
                    ((3, 200, 72), (3, 196, 72)), ((4, 50, 36), (1, 44, 36)), ((16, 128, 128), (128, 128)),
                    ((2, 3, 64, 32), (2, 3, 80, 32)), ((2, 3, 64, 32), (2, 1, 80, 32)), ((2048, 128), (512, 128))]


@pytest.mark.parametrize("xs,ys", TRANSPOSED_CASES)
def test_nt_product_reads_the_transposed_operand_in_place(xs, ys):
    """x @ y^T with y stored (.., N, K): the same bits as permute + matmul, and 1e-4 of float64."""
    require_gpu()
    x, y = f32(*xs), f32(*ys, scale=xs[-1] ** -0.5)
    xd, yd = dev(x), dev(y)
    got = xd.matmul_nt(yd).numpy()
    nd = yd.ndim
    check(got, xd.matmul(yd.transpose(nd - 2, nd - 1)).numpy(), 0, f"NT {xs} {ys} vs permute + NN")
    check_mm(got, x.astype(np.float64) @ np.swapaxes(y.astype(np.float64), -1, -2), f"NT {xs} {ys}")


@pytest.mark.parametrize("xs,ys", TRANSPOSED_CASES)
def test_tn_product_reads_the_transposed_operand_in_place(xs, ys):
    """x^T @ y with x stored (.., K, M); shapes are the NT cases with both operands swapped around."""
    require_gpu()
    xs, ys = xs[:-2] + (xs[-1], xs[-2]), ys[:-2] + (ys[-1], ys[-2])          # (.., K, M), (.., K, N)
    x, y = f32(*xs), f32(*ys, scale=xs[-2] ** -0.5)
    xd, yd = dev(x), dev(y)
    got = xd.matmul_tn(yd).numpy()
    nd = xd.ndim
    check(got, xd.transpose(nd - 2, nd - 1).matmul(yd).numpy(), 0, f"TN {xs} {ys} vs permute + NN")
    check_mm(got, np.swapaxes(x.astype(np.float64), -1, -2) @ y.astype(np.float64), f"TN {xs} {ys}")


@pytest.mark.parametrize("tile", list(__import__("dlgrad_amd.codegen.hip_kernel", fromlist=["x"]).MATMUL_CONFIGS))
def test_every_tile_configuration_transposed(tile, monkeypatch):
    require_gpu()
    from dlgrad_amd.runtime.hip import HIP
    x, y, z = f32(2, 260, 72), f32(2, 388, 72, scale=72 ** -0.5), f32(2, 260, 100)
    xd, yd, zd = dev(x), dev(y), dev(z)
    monkeypatch.setattr(HIP, "MATMUL_FORCE", "64x64")
    want_nt, want_tn = xd.matmul(yd.transpose(1, 2)).numpy(), xd.transpose(1, 2).matmul(zd).numpy()
    monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
    check(xd.matmul_nt(yd).numpy(), want_nt, 0, f"NT {tile}")
    check(xd.matmul_tn(zd).numpy(), want_tn, 0, f"TN {tile}")


@pytest.mark.parametrize("T,d,batch", [(128, 32, (2, 3)), (1024, 64, (2,)), (100, 20, (3,)), (257, 64, ()), (64, 8, (1, 2))])
def test_triangular_hints_skip_work_without_changing_a_bit(T, d, batch, monkeypatch):
    """tri = out_lower / a_lower / at_lower tell the product kernel which tiles or which part of
    the k range a triangular operand or a masked consumer makes irrelevant.  With operands that
    really have that structure every kept entry must equal the plain product bit for bit, for
    every tile configuration (forced one by one), ragged T included."""
    require_gpu()
    from dlgrad_amd.codegen import hip_kernel as K
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_SPLITK", False)     # the plain products compared with are the unsplit kernel's (a split-k tile adds slice sums)
    rng = np.random.default_rng(T + d)
    low = np.tril(rng.standard_normal(batch + (T, T), dtype=np.float32))          # zero above the diagonal
    x = rng.standard_normal(batch + (T, d), dtype=np.float32)
    y = rng.standard_normal(batch + (T, d), dtype=np.float32)
    keep = np.tril(np.ones((T, T), bool))
    lowd, xd, yd = dev(low), dev(x), dev(y)
    want_scores = xd.matmul_nt(yd).numpy()
    want_av = lowd.matmul(yd).numpy()
    want_atv = lowd.matmul_tn(yd).numpy()
    tiles = [t for t in K.MATMUL_CONFIGS if T >= 64 or t in K.MATMUL_SMALL_TILES]
    for tile in tiles:
        prev, HIP.MATMUL_FORCE = HIP.MATMUL_FORCE, tile
        try:
            got = xd.matmul_nt(yd, tri="out_lower").numpy()
            if not hip.COMPILE_ONLY:
                assert (got[..., keep].view(np.uint32) == want_scores[..., keep].view(np.uint32)).all(), f"out_lower {tile}"
            check(lowd.matmul(yd, tri="a_lower").numpy(), want_av, 0, f"a_lower {tile}")
            check(lowd.matmul_tn(yd, tri="at_lower").numpy(), want_atv, 0, f"at_lower {tile}")
        finally:
            HIP.MATMUL_FORCE = prev


@pytest.mark.parametrize("shape_x,shape_y,nt", [((256, 96), (96, 128), False), ((3, 100, 36), (50, 36), True),
                                                ((2, 3, 65, 17), (2, 3, 17, 33), False), ((512, 384), (1536, 384), True),
                                                ((4, 0), (0, 8), False)])
def test_epilogues_equal_the_separate_elementwise_kernels(shape_x, shape_y, nt):
    """epi = add / relu / gate do their one fp32 operation on the accumulator as it is stored: the bits
    of product + e, relu(product) and where(e > 0, product, 0) computed by separate kernels, for
    every tile configuration (forced one by one), ragged and batched shapes, NN and NT, empty k."""
    require_gpu()
    from dlgrad_amd.codegen import hip_kernel as K
    from dlgrad_amd.runtime.hip import HIP
    rng = np.random.default_rng(len(shape_x) * 1000 + shape_x[-1])
    x = rng.standard_normal(shape_x, dtype=np.float32)
    y = rng.standard_normal(shape_y, dtype=np.float32)
    xd, yd = dev(x), dev(y)
    mm = (lambda **kw: xd.matmul_nt(yd, **kw)) if nt else (lambda **kw: xd.matmul(yd, **kw))
    plain = mm()
    e = rng.standard_normal(plain.shape, dtype=np.float32)
    e[..., ::3] = 0.0                                                 # gate: zero is not positive
    ed = dev(e)
    want_add = (plain + ed).numpy()
    want_relu = plain.relu().numpy()
    want_gate = (ed > 0.0).where(inp=plain, other=0.0).numpy()
    bias = rng.standard_normal((1, plain.shape[-1]), dtype=np.float32)           # one row, added to every row of the product
    bd = dev(bias)
    want_bias = (plain + bd).numpy()
    small = min(plain.shape[-2:]) < 64
    tiles = [None] + [t for t in K.MATMUL_CONFIGS if not small or t in K.MATMUL_SMALL_TILES]
    for tile in tiles:
        prev, HIP.MATMUL_FORCE = HIP.MATMUL_FORCE, tile
        try:
            check(mm(epi="add", e=ed).numpy(), want_add, 0, f"add {tile}")
            check(mm(epi="relu").numpy(), want_relu, 0, f"relu {tile}")
            check(mm(epi="gate", e=ed).numpy(), want_gate, 0, f"gate {tile}")
            check(mm(epi="bias", e=bd).numpy(), want_bias, 0, f"bias {tile}")
        finally:
            HIP.MATMUL_FORCE = prev


def test_epilogues_are_refused_without_a_fitting_operand():
    require_gpu()
    a, b = dev(f32(8, 16)), dev(f32(16, 8))
    with pytest.raises(ValueError):
        a.matmul(b, epi="add")                          # nothing to add
    with pytest.raises(ValueError):
        a.matmul(b, epi="gate", e=dev(f32(8, 4)))       # wrong size
    with pytest.raises(ValueError):
        a.matmul(b, epi="bias", e=dev(f32(8, 8)))       # a bias is one row
    with pytest.raises(ValueError):
        a.matmul(b, epi="square")                       # no such step
    with pytest.raises(ValueError):
        a.matmul_nt(dev(f32(8, 16)), tri="out_lower", epi="relu")


def test_triangular_hints_are_refused_where_they_make_no_sense():
    require_gpu()
    a, b = dev(f32(8, 16)), dev(f32(16, 8))
    with pytest.raises(ValueError):
        a.matmul(b, tri="a_lower")                      # A is not square
    with pytest.raises(ValueError):
        a.matmul_nt(dev(f32(4, 16)), tri="out_lower")   # the output is not square


@pytest.mark.parametrize("N,K,lead", [(128, 128, (1, 1)), (384, 128, (1,)), (65, 128, ()), (512, 2048, (1, 1)), (7, 12, (1,)), (130, 1000, ())])
def test_one_row_times_a_transposed_matrix(N, K, lead, monkeypatch):
    """The linear layers of a decoding step, x (1, K) against W (N, K): one wavefront per output
    instead of an MFMA tile with one useful row.  Checked against float64 and against the tile path
    (1e-6 of the largest entry: the k sum is split over the lanes), with each epilogue."""
    require_gpu()
    from dlgrad_amd.runtime.hip import HIP
    rng = np.random.default_rng(N + K)
    x = rng.standard_normal(lead + (1, K), dtype=np.float32)
    w = rng.standard_normal((N, K), dtype=np.float32)
    e = rng.standard_normal(lead + (1, N), dtype=np.float32)
    e[..., ::3] = 0.0
    xd, wd, ed = dev(x), dev(w), dev(e)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    variants = {"": want, "add": want + e, "relu": np.maximum(want, 0), "gate": np.where(e > 0, want, 0)}
    for epi, ref in variants.items():
        kw = {"epi": epi, "e": ed} if epi in ("add", "gate") else {"epi": epi} if epi else {}
        before = hip.launch_count
        got = xd.matmul_nt(wd, **kw).numpy()
        assert hip.launch_count - before == 1
        monkeypatch.setattr(HIP, "ROW_MATMUL", False)
        tiled = xd.matmul_nt(wd, **kw).numpy()
        monkeypatch.setattr(HIP, "ROW_MATMUL", True)
        if hip.COMPILE_ONLY:
            continue
        assert got.shape == ref.shape
        top = np.abs(want).max()
        assert np.abs(got - ref).max() <= 2e-6 * top, f"{epi or 'plain'} vs float64"
        assert np.abs(got - tiled).max() <= 2e-6 * top, f"{epi or 'plain'} vs the tile path"


def _rows_vs_float64(got: np.ndarray, rows: np.ndarray, a_rows: np.ndarray, b: np.ndarray, what: str) -> None:
    """`got[rows]` against the float64 product of the matching rows of the left operand: a full
    float64 product of these sizes is a teraflop on the host, a sample of rows (spread over
    every tile row, all columns) is not."""
    if hip.COMPILE_ONLY:
        return
    want = a_rows.astype(np.float64) @ b.astype(np.float64)
    err = np.abs(got[rows] - want).max() / (np.abs(want).max() + 1e-30)
    assert err <= 1e-4, f"{what}: {err:.3e}"
    assert np.isfinite(got).all(), what


def test_8192_cubed_against_float64_on_a_row_sample():
    require_gpu()
    n = 8192
    rng = np.random.default_rng(31)
    x = rng.standard_normal((n, n), dtype=np.float32)
    y = rng.standard_normal((n, n), dtype=np.float32) * np.float32(n ** -0.5)
    got = (dev(x) @ dev(y)).numpy()
    rows = np.unique(np.concatenate([np.arange(0, n, 67), [n - 1]]))        # every 256-row tile is hit
    _rows_vs_float64(got, rows, x[rows], y, "8192^3")
    if not hip.COMPILE_ONLY:                                                # linearity: (x @ y) 1 = x (y 1), every row
        lhs = got.astype(np.float64).sum(1)
        rhs = x.astype(np.float64) @ y.astype(np.float64).sum(1)
        assert np.abs(lhs - rhs).max() <= 1e-4 * np.abs(rhs).max() + 1e-3


def test_4096_backward_shapes_in_place_against_float64_on_a_row_sample():
    """A^T G (TN kernel) and G B^T (NT kernel) at the benchmark's 4096 size, and the same two
    products as the reference issues them (materialised transpose, then NN)."""
    require_gpu()
    n = 4096
    rng = np.random.default_rng(32)
    a = rng.standard_normal((n, n), dtype=np.float32) * np.float32(n ** -0.5)
    g = rng.standard_normal((n, n), dtype=np.float32) * np.float32(n ** -0.5)
    da, dg = dev(a), dev(g)
    rows = np.unique(np.concatenate([np.arange(0, n, 61), [n - 1]]))
    tn = da.matmul_tn(dg).numpy()                                           # a^T g
    _rows_vs_float64(tn, rows, np.ascontiguousarray(a.T[rows]), g, "4096 TN in place")
    nt = dg.matmul_nt(da).numpy()                                           # g a^T
    _rows_vs_float64(nt, rows, g[rows], np.ascontiguousarray(a.T), "4096 NT in place")
    check(((da.T) @ dg).numpy(), tn, 0, "permute + NN gives the TN kernel's bits")
    check((dg @ da.T).numpy(), nt, 0, "permute + NN gives the NT kernel's bits")


PAIR_CASES = [
    # (shape of g, shape of w, shape of x, epilogue of the first product)
    ((16, 128, 128), (128, 128), (16, 128, 128), ""),          # the attention projection of the char-GPT step
    ((16, 128, 384), (384, 128), (16, 128, 128), ""),          # its stacked q/k/v projection
    ((16, 128, 128), (128, 512), (16, 128, 512), "gate"),      # its feed-forward block: hidden gradient with the ReLU select
    ((16, 128, 512), (512, 128), (16, 128, 128), ""),
    ((3, 50, 36), (36, 20), (3, 50, 20), ""),                  # extents that are no multiple of a tile
    ((2, 33, 7), (7, 5), (2, 33, 5), "gate"),                  # 4-byte accesses
    ((1, 1, 64), (64, 32), (1, 1, 32), ""),                    # a single row
    ((256, 64), (64, 10), (256, 10), "relu"),                  # 2-D operands (the MLP)
]


@pytest.mark.parametrize("gs,ws,xs,epi", PAIR_CASES)
def test_two_products_in_one_launch_keep_their_bits(gs, ws, xs, epi, monkeypatch):
    """dX = G W (optionally with an epilogue) and dW = G^T X of a linear layer go out as one launch of two
    tile grids.  Each block runs the product kernel's own code on the block index it would have had, so both
    results must equal those of the separate launches bit for bit, and the pair must be one launch.  (The separate
    launches are held to the tiles that add k in one piece: a product alone may otherwise be given a tile that cuts k
    into slices, which a pair never is.)"""
    require_gpu()
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_SPLITK", False)
    rng = np.random.default_rng(91)
    g, w, x = (rng.standard_normal(s, dtype=np.float32) for s in (gs, ws, xs))
    gate = rng.standard_normal(gs[:-1] + ws[-1:], dtype=np.float32)
    gb, wb, xb, eb = (dev(a) for a in (g, w, x, gate))
    first = ("nn", gb, wb, epi, eb if epi != "relu" else None) if epi else ("nn", gb, wb)
    before = hip.launch_count
    dx, dw = Buffer.matmul_pair(first, ("tn", gb, xb))
    launches = hip.launch_count - before
    kw = {"epi": epi, "e": eb if epi != "relu" else None} if epi else {}
    dx0, dw0 = gb.matmul(wb, **kw), gb.matmul_tn(xb)
    assert dx.shape == dx0.shape and dw.shape == dw0.shape
    if hip.COMPILE_ONLY:
        return
    if gs[-2] > 1:
        assert launches == 1, launches
    np.testing.assert_array_equal(dx.numpy().view(np.uint32), dx0.numpy().view(np.uint32))
    np.testing.assert_array_equal(dw.numpy().view(np.uint32), dw0.numpy().view(np.uint32))
    want = (g.astype(np.float64) @ w.astype(np.float64))
    if epi == "gate":
        want = np.where(gate > 0, want, 0.0)
    elif epi == "relu":
        want = np.maximum(want, 0.0)
    check_mm(dx.numpy(), want, "dx against float64")
    want_w = np.swapaxes(g.astype(np.float64), -1, -2) @ x.astype(np.float64)
    check_mm(dw.numpy(), want_w, "dw against float64")


def test_large_products_do_not_travel_in_pairs():
    """Beyond about a GFLOP a product fills the chip by itself: the pair entry then issues two launches
    (and gives the same bits, being the same two calls)."""
    require_gpu()
    from dlgrad_amd.buffer import Buffer
    rng = np.random.default_rng(92)
    g, w, x = (rng.standard_normal(s, dtype=np.float32) for s in ((4, 1024, 512), (512, 384), (4, 1024, 384)))
    gb, wb, xb = dev(g), dev(w), dev(x)
    before = hip.launch_count
    dx, dw = Buffer.matmul_pair(("nn", gb, wb), ("tn", gb, xb))
    assert hip.launch_count - before == 2
    if hip.COMPILE_ONLY:
        return
    np.testing.assert_array_equal(dx.numpy().view(np.uint32), gb.matmul(wb).numpy().view(np.uint32))
    np.testing.assert_array_equal(dw.numpy().view(np.uint32), gb.matmul_tn(xb).numpy().view(np.uint32))


@pytest.mark.parametrize("K_,N,epi", [(128, 384, ""), (128, 512, "relu"), (128, 65, ""), (512, 128, "add"), (768, 7, ""), (1024, 260, "relu"),
                                      (36, 20, "add")])
def test_single_row_product_normalises_its_row_on_the_way(K_, N, epi):
    """Decoding: RMSNorm followed by a linear layer on one row runs as one launch -- every wavefront of the
    single-row product normalises the row for itself, with the statements of the RMSNorm kernel.  The result
    must have the bits of the two launches, and be the float64 value to 2e-6 of the largest entry."""
    require_gpu()
    from dlgrad_amd import Tensor, nn
    rng = np.random.default_rng(93)
    x = rng.standard_normal((1, 1, K_), dtype=np.float32) * 3
    w = rng.standard_normal((N, K_), dtype=np.float32) * K_ ** -0.5
    gain = (1 + 0.1 * rng.standard_normal((1, K_))).astype(np.float32)
    res = rng.standard_normal((1, 1, N), dtype=np.float32)
    norm = nn.RMSNorm(K_, device="hip")
    norm.weight = Tensor(gain, device="hip", requires_grad=True)
    xt, wb, rb = Tensor(x, device="hip"), dev(w), dev(res)
    assert hip.HIP.row_norm_fits(xt.data, wb, norm.weight.data)
    kw = {"epi": epi, "e": rb if epi == "add" else None} if epi else {}
    before = hip.launch_count
    fused = xt.data.matmul_nt(wb, norm=(norm.weight.data, norm.eps), **kw)
    assert hip.launch_count - before == 1
    two = norm(xt).data.matmul_nt(wb, **kw)
    if hip.COMPILE_ONLY:
        return
    np.testing.assert_array_equal(fused.numpy().view(np.uint32), two.numpy().view(np.uint32))
    x64 = x.astype(np.float64)
    y64 = (x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + norm.eps) * gain) @ w.T.astype(np.float64)
    y64 = np.maximum(y64, 0) if epi == "relu" else y64 + res if epi == "add" else y64
    assert np.abs(fused.numpy() - y64).max() <= 2e-6 * max(1.0, np.abs(y64).max())


def test_rows_the_normalising_product_does_not_take():
    require_gpu()
    from dlgrad_amd.runtime.hip import HIP
    g = lambda k: dev(np.ones((1, k), np.float32))                                      # noqa: E731
    x = lambda *s: dev(np.ones(s, np.float32))                                          # noqa: E731
    assert HIP.row_norm_fits(x(1, 1, 128), x(64, 128), g(128))
    assert not HIP.row_norm_fits(x(1, 2, 128), x(64, 128), g(128))                      # two rows
    assert not HIP.row_norm_fits(x(1, 1, 130), x(64, 130), g(130))                      # rows that are no whole 16-byte items
    assert not HIP.row_norm_fits(x(1, 1, 2048), x(8, 2048), g(2048))                    # a row beyond the registers kept for it
    assert not HIP.row_norm_fits(x(1, 1, 128), x(2, 64, 128), g(128))                   # a batch of matrices
    assert HIP.tile_norm_fits(x(1, 2, 128), x(64, 128), g(128))                         # several rows: the tile product takes them,
    assert not HIP.tile_norm_fits(x(4, 256), x(64, 256), g(256))                        # up to 128 floats a row
    assert not HIP.tile_norm_fits(x(4, 128), x(2, 64, 128), g(128))
    with pytest.raises(ValueError):
        x(1, 2, 130).matmul_nt(x(64, 130), norm=(g(130), 1e-6))


@pytest.mark.parametrize("xs,N,epi,tile", [((16, 128, 128), 384, "", ""), ((16, 128, 128), 512, "relu", ""), ((1, 128, 128), 65, "", ""),
                                           ((3, 50, 36), 20, "add", ""), ((2048, 128), 128, "", "64x64m16k128"), ((70, 64), 260, "relu", "32x32m16k128"),
                                           ((1, 1, 128), 384, "", "32x32m16k128")])
def test_tile_product_normalises_the_rows_of_its_left_operand(xs, N, epi, tile, monkeypatch):
    """RMSNorm followed by a linear layer as one launch for rows of up to 128 floats: a block's tile of x holds whole
    rows (one k step), which its wavefronts normalise in LDS with the statements of the RMSNorm kernel before the
    matrix steps begin.  Result, normalised rows and 1 / rms must have the bits of the two launches."""
    require_gpu()
    from dlgrad_amd import Tensor, nn
    from dlgrad_amd.runtime.hip import HIP
    if tile:
        monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
    rng = np.random.default_rng(94)
    Kd = xs[-1]
    x = rng.standard_normal(xs, dtype=np.float32) * 2
    w = rng.standard_normal((N, Kd), dtype=np.float32) * Kd ** -0.5
    gain = (1 + 0.1 * rng.standard_normal((1, Kd))).astype(np.float32)
    res = rng.standard_normal(xs[:-1] + (N,), dtype=np.float32)
    xb, wb, gb, rb = dev(x), dev(w), dev(gain), dev(res)
    assert HIP.tile_norm_fits(xb, wb, gb)
    kw = {"epi": epi, "e": rb if epi == "add" else None} if epi else {}
    before = hip.launch_count
    out, yn, rinv = xb.matmul_nt(wb, norm=(gb, 1e-6, True), **kw)
    assert hip.launch_count - before == 1 and "_rms" in (HIP.last_matmul_kernel or "_rms")
    only = xb.matmul_nt(wb, norm=(gb, 1e-6), **kw) if x.size > Kd else out               # (a single row takes the row kernel)
    y2, r2 = xb.rmsnorm(gb, 1e-6)
    out2 = y2.matmul_nt(wb, **kw)
    assert out.shape == out2.shape and yn.shape == y2.shape and rinv.shape == r2.shape
    if hip.COMPILE_ONLY:
        return
    for name, a, b in (("result", out, out2), ("result alone", only, out2), ("normalised rows", yn, y2), ("1 / rms", rinv, r2)):
        np.testing.assert_array_equal(a.numpy().view(np.uint32), b.numpy().view(np.uint32), err_msg=name)
    x64 = x.astype(np.float64)
    y64 = (x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6) * gain) @ w.T.astype(np.float64)
    y64 = np.maximum(y64, 0) if epi == "relu" else y64 + res if epi == "add" else y64
    check_mm(out.numpy(), y64, "against float64")


@pytest.mark.parametrize("tile", ["128x128/4", "64x64k64/8", "64x64m16/3", "128x64/2", "64x64k64/16"])
def test_split_k_products_add_their_slices_in_a_fixed_order(tile, monkeypatch):
    """The k sum cut into slices, one block per (tile, slice), the partial tiles added up by a column-sum
    launch: NN, TN and NT forms, edge tiles, a k that the slices do not divide, batches -- against float64 at
    the product bar of 1e-4 (the bits are not those of the unsplit kernel: an element is now a sum of
    per-slice sums), and the same bits on a repeat."""
    require_gpu()
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
    for (M, Kd, N), batch in (((512, 512, 512), ()), ((200, 1030, 136), ()), ((96, 2048, 520), ()), ((130, 700, 70), (3,)),
                              ((64, 4096, 64), (2, 2)), ((1024, 1024, 1024), ())):
        a, b = f32(*batch, M, Kd), f32(*batch, Kd, N, scale=Kd ** -0.5)
        da, db = dev(a), dev(b)
        first = da.matmul(db).numpy()
        if not hip.COMPILE_ONLY:
            assert "_sk" in HIP.last_matmul_kernel.split("_w")[1], HIP.last_matmul_kernel    # (then _d: the deep k loop; _x: whole tiles, no bounds tests)
        check_mm(first, a.astype(np.float64) @ b.astype(np.float64), f"{tile} {batch}{(M, Kd, N)}")
        again = da.matmul(db).numpy()
        if not hip.COMPILE_ONLY:
            np.testing.assert_array_equal(again, first, err_msg=f"{tile} {(M, Kd, N)} repeated")
        if not batch:
            at, bt = dev(np.ascontiguousarray(a.T)), dev(np.ascontiguousarray(b.T))
            check_mm(at.matmul_tn(db).numpy(), a.astype(np.float64) @ b.astype(np.float64), f"{tile} TN {(M, Kd, N)}")
            check_mm(da.matmul_nt(bt).numpy(), a.astype(np.float64) @ b.astype(np.float64), f"{tile} NT {(M, Kd, N)}")
    # an epilogue cannot be split: the forced tile falls back to its unsplit form and the bits are the unsplit kernel's
    a, b, e = f32(128, 512), f32(512, 128, scale=512 ** -0.5), f32(128, 128)
    fused = dev(a).matmul(dev(b), epi="add", e=dev(e)).numpy()
    monkeypatch.setattr(HIP, "MATMUL_FORCE", tile.split("/")[0])
    if not hip.COMPILE_ONLY:
        np.testing.assert_array_equal(fused, ((dev(a) @ dev(b)) + dev(e)).numpy())


@pytest.mark.parametrize("tile", ["64x64k64*2", "64x64k32*4", "32x32m16*4", "32x32*8", "128x128*2", "64x64*3"])
def test_k_group_products_add_their_slices_in_a_fixed_order(tile, monkeypatch):
    """The k sum cut among groups of wavefronts inside every block, the partial tiles joined through LDS in group
    order: NN, TN and NT forms, edge tiles, a k that the groups do not divide (the last group's extra steps read
    zeros), batches -- against float64 at the product bar of 1e-4, and the same bits on a repeat."""
    require_gpu()
    from dlgrad_amd.runtime.hip import HIP
    monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
    for (M, Kd, N), batch in (((512, 512, 512), ()), ((200, 1030, 136), ()), ((96, 2048, 520), ()), ((130, 700, 70), (3,)),
                              ((64, 4096, 64), (2, 2)), ((1024, 1024, 1024), ()), ((64, 96, 64), ())):
        a, b = f32(*batch, M, Kd), f32(*batch, Kd, N, scale=Kd ** -0.5)
        da, db = dev(a), dev(b)
        first = da.matmul(db).numpy()
        if not hip.COMPILE_ONLY:
            assert f"_g{HIP._group_plan(tile, Kd)[0]}" in HIP.last_matmul_kernel, HIP.last_matmul_kernel
        check_mm(first, a.astype(np.float64) @ b.astype(np.float64), f"{tile} {batch}{(M, Kd, N)}")
        again = da.matmul(db).numpy()
        if not hip.COMPILE_ONLY:
            np.testing.assert_array_equal(again, first, err_msg=f"{tile} {(M, Kd, N)} repeated")
        if not batch:
            at, bt = dev(np.ascontiguousarray(a.T)), dev(np.ascontiguousarray(b.T))
            check_mm(at.matmul_tn(db).numpy(), a.astype(np.float64) @ b.astype(np.float64), f"{tile} TN {(M, Kd, N)}")
            check_mm(da.matmul_nt(bt).numpy(), a.astype(np.float64) @ b.astype(np.float64), f"{tile} NT {(M, Kd, N)}")
    # an epilogue takes no k-group tile: the forced tile falls back to its plain form and the bits are the plain kernel's
    a, b, e = f32(128, 512), f32(512, 128, scale=512 ** -0.5), f32(128, 128)
    fused = dev(a).matmul(dev(b), epi="add", e=dev(e)).numpy()
    monkeypatch.setattr(HIP, "MATMUL_FORCE", tile.split("*")[0])
    if not hip.COMPILE_ONLY:
        np.testing.assert_array_equal(fused, ((dev(a) @ dev(b)) + dev(e)).numpy())


def test_two_step_deep_k_loop_gives_the_bits_of_the_plain_loop(monkeypatch):
    """The k loop that fetches two steps ahead and issues its fetches and LDS stores between the MFMA steps performs the
    loads and MFMA steps of the plain loop in the same order: same bits, for every tile -- on a shape with edge tiles
    and a ragged k (the guarded form), on whole tiles (the form without bounds tests), with one, two and three k steps,
    as stored and transposed in place, with epilogues, triangular structure, split k and k groups."""
    require_gpu()
    from dlgrad_amd.codegen import hip_kernel as K
    from dlgrad_amd.runtime.hip import HIP
    rng = np.random.default_rng(12)

    def both(run, what):
        monkeypatch.setattr(HIP, "MATMUL_DEEP", False)
        want = run().numpy()
        plain = HIP.last_matmul_kernel
        monkeypatch.setattr(HIP, "MATMUL_DEEP", True)
        got = run().numpy()
        if not hip.COMPILE_ONLY:
            assert plain and "_d" not in plain.split("_w")[1] and "_d" in HIP.last_matmul_kernel.split("_w")[1], (what, plain, HIP.last_matmul_kernel)
        check(got, want, 0, f"{what}: deep loop vs plain loop")

    for tile, cfg in K.MATMUL_CONFIGS.items():
        bm, bn, _ = K.matmul_tile_shape(tile)
        monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
        for M, N, Kd in ((200, 196, 328), (2 * bm, 2 * bn, 3 * cfg[4]), (bm, bn, cfg[4]), (bm + 4, bn, 2 * cfg[4] + 8)):
            x, y = rng.standard_normal((M, Kd), dtype=np.float32), rng.standard_normal((Kd, N), dtype=np.float32) * np.float32(Kd ** -0.5)
            e = rng.standard_normal((M, N), dtype=np.float32)
            xd, yd, ytd, xtd, ed = dev(x), dev(y), dev(np.ascontiguousarray(y.T)), dev(np.ascontiguousarray(x.T)), dev(e)
            both(lambda: xd.matmul(yd), f"{tile} {(M, N, Kd)} nn")
            both(lambda: xd.matmul_nt(ytd), f"{tile} {(M, N, Kd)} nt")
            both(lambda: xtd.matmul_tn(yd), f"{tile} {(M, N, Kd)} tn")
            both(lambda: xd.matmul(yd, epi="add", e=ed), f"{tile} {(M, N, Kd)} nn add")
            both(lambda: xd.matmul_nt(ytd, epi="gate", e=ed), f"{tile} {(M, N, Kd)} nt gate")
        T = 2 * max(bm, bn) + 8
        q, kk = rng.standard_normal((2, T, 64), dtype=np.float32), rng.standard_normal((2, T, 64), dtype=np.float32)
        low = np.tril(rng.standard_normal((2, T, T), dtype=np.float32))
        qd, kd, lowd = dev(q), dev(kk), dev(low)
        both(lambda: qd.matmul_nt(kd, tri="out_lower"), f"{tile} out_lower")
        both(lambda: lowd.matmul(kd, tri="a_lower"), f"{tile} a_lower")
        both(lambda: lowd.matmul_tn(kd, tri="at_lower"), f"{tile} at_lower")
    x, y = rng.standard_normal((200, 1030), dtype=np.float32), rng.standard_normal((1030, 136), dtype=np.float32)
    xd, yd = dev(x), dev(y)
    for tile in ("128x128/4", "64x64k64/8", "64x64k64*2", "32x32m16*4", "64x64k32*4"):
        monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
        both(lambda: xd.matmul(yd), f"{tile} ragged")
    x, y = rng.standard_normal((256, 1024), dtype=np.float32), rng.standard_normal((1024, 256), dtype=np.float32)
    xd, yd = dev(x), dev(y)
    for tile in ("128x128/4", "64x64k64/8", "64x64k64*2", "32x32m16*4", "64x64k32*4"):
        monkeypatch.setattr(HIP, "MATMUL_FORCE", tile)
        both(lambda: xd.matmul(yd), f"{tile} whole tiles")

