"""Pins the C restatement (oracle/) against independent statements of each result:
numpy broadcasting / float64 maths / brute force -- never the oracle's own formula.
CPU only."""
import numpy as np
import pytest

from oracle import cref

RNG = np.random.default_rng(7)


def f32(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


# the reference's own broadcast matrix (test/test_ops.py:29-43): every 1|d combination
def bcast_cases(shape):
    out = []
    for mask in range(2 ** len(shape)):
        out.append(tuple(1 if (mask >> i) & 1 else d for i, d in enumerate(shape)))
    return out


@pytest.mark.parametrize("op,npop", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply)])
@pytest.mark.parametrize("shape", [(2, 3, 4, 5), (2, 3, 4), (78, 64), (7,)])
def test_arithmetic_bit_exact(op, npop, shape):
    x = f32(*shape)
    for ys in bcast_cases(shape):
        y = f32(*ys)
        np.testing.assert_array_equal(cref.binary(op, x, y), npop(x, y))


def test_arithmetic_lower_rank_operand():
    x = f32(3, 4, 5)
    y = f32(4, 5)
    z = f32(5)
    s = np.float32(1.75)
    np.testing.assert_array_equal(cref.binary("add", x, y), x + y)
    np.testing.assert_array_equal(cref.binary("mul", x, z), x * z)
    np.testing.assert_array_equal(cref.binary("sub", x, s), x - s)
    np.testing.assert_array_equal(cref.binary("mul", np.float32(3), np.float32(4)), np.float32(12))


def test_div_within_one_ulp():
    x, y = f32(64, 33), f32(64, 33)
    got, want = cref.binary("div", x, y), x / y
    assert np.all(np.abs(got - want) <= np.spacing(np.abs(want)))
    got = cref.binary("div", x, f32(64, 1) + 3)
    assert got.shape == (64, 33)


@pytest.mark.parametrize("op,npop", [("eq", np.equal), ("gt", np.greater), ("gte", np.greater_equal),
                                     ("lt", np.less)])
def test_comparisons(op, npop):
    x = RNG.integers(-2, 3, (6, 7)).astype(np.float32)
    y = RNG.integers(-2, 3, (6, 7)).astype(np.float32)
    np.testing.assert_array_equal(cref.binary(op, x, y), npop(x, y).astype(np.float32))
    np.testing.assert_array_equal(cref.binary(op, x, np.float32(0)), npop(x, 0).astype(np.float32))


def test_cmp_le_is_tril_mask():
    H, W = 5, 7
    cols = np.arange(W, dtype=np.float32).reshape(1, W)
    rows = np.arange(H, dtype=np.float32).reshape(H, 1)
    got = cref.cmp_le(cols, rows, (H, W))
    np.testing.assert_array_equal(got, np.tril(np.ones((H, W), np.float32)))


def test_unary_against_float64():
    x = f32(1000)
    pos = np.abs(x) + np.float32(1e-3)
    np.testing.assert_array_equal(cref.unary("neg", x), -x)
    for op, fn, arg in (("exp", np.exp, x), ("log", np.log, pos), ("sqrt", np.sqrt, pos),
                        ("rsqrt", lambda v: 1 / np.sqrt(v), pos)):
        want = fn(arg.astype(np.float64))
        got = cref.unary(op, arg).astype(np.float64)
        assert np.max(np.abs(got - want) / np.abs(want)) < 3e-7, op   # fast-math sqrt/div: ~2 ulp


@pytest.mark.parametrize("n", [2, 3, -1, 0, 5, 2.9])
def test_pow_truncates_exponent(n):
    x = np.abs(f32(257)) + 0.5
    want = x.astype(np.float64) ** int(n)          # int(2.9) == 2: the quirk
    got = cref.unary("pow", x, n)
    np.testing.assert_allclose(got, want, rtol=3e-7)


def test_relu_and_clamp():
    x = f32(100)
    np.testing.assert_array_equal(cref.unary("relu", x), np.maximum(x, 0))
    np.testing.assert_array_equal(cref.clamp(x, -0.5, 0.25), np.clip(x, -0.5, 0.25))
    np.testing.assert_array_equal(cref.clamp(x, 0, None), np.maximum(x, 0))
    np.testing.assert_array_equal(cref.clamp(x, None, 0.1), np.minimum(x, np.float32(0.1)))
    np.testing.assert_array_equal(cref.clamp(x), x)


@pytest.mark.parametrize("shape", [(5,), (4, 7), (3, 4, 5), (2, 3, 4, 5), (64, 1000)])
def test_reductions(shape):
    x = f32(*shape)
    x64 = x.astype(np.float64)
    np.testing.assert_allclose(cref.reduce("sum", x), x64.sum(), rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(cref.reduce("mean", x), x64.mean(), rtol=1e-5, atol=1e-6)
    assert cref.reduce("max", x) == x.max()
    for d in range(len(shape)):
        np.testing.assert_allclose(cref.reduce("sum", x, d), x64.sum(axis=d), rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(cref.reduce("mean", x, d), x64.mean(axis=d), rtol=1e-5, atol=1e-5)
        np.testing.assert_array_equal(cref.reduce("max", x, d), x.max(axis=d))


def test_sum_of_known_series():
    # closed form: 1..n sums to n(n+1)/2 exactly in fp32 for n = 2000
    x = np.arange(1, 2001, dtype=np.float32).reshape(40, 50)
    assert cref.reduce("sum", x) == 2000 * 2001 / 2
    np.testing.assert_array_equal(cref.reduce("sum", x, 0), x.astype(np.float64).sum(0))


def test_max_all_below_minus_flt_max_start():
    x = np.full((3, 4), -np.inf, np.float32)
    # the kernels start from -FLT_MAX, so an all -inf row reports -FLT_MAX
    assert cref.reduce("max", x) == -np.finfo(np.float32).max
    np.testing.assert_array_equal(cref.reduce("max", x, 1), np.full(3, -np.finfo(np.float32).max, np.float32))


def test_argmax_first_index_on_ties():
    x = f32(6, 9)
    np.testing.assert_array_equal(cref.argmax(x, 1), x.argmax(1).astype(np.float32))
    np.testing.assert_array_equal(cref.argmax(x, 0), x.argmax(0).astype(np.float32))
    np.testing.assert_array_equal(cref.argmax(x, None), [np.float32(x.argmax())])
    t = np.zeros((3, 8), np.float32)
    t[0, [2, 5]] = 4.0
    t[1, :] = 1.0
    t[2, [7, 3]] = 9.0
    np.testing.assert_array_equal(cref.argmax(t, 1), [2, 0, 3])
    np.testing.assert_array_equal(cref.argmax(t.T.copy(), 0), [2, 0, 3])


@pytest.mark.parametrize("shape,order", [((4, 7), (1, 0)), ((2, 3, 4), (0, 2, 1)), ((2, 3, 4), (2, 0, 1)),
                                         ((2, 3, 4, 5), (0, 2, 1, 3)), ((2, 3, 4, 5), (0, 1, 3, 2)),
                                         ((2, 3, 4, 5), (3, 2, 1, 0)), ((5,), (0,))])
def test_permute(shape, order):
    x = f32(*shape)
    np.testing.assert_array_equal(cref.permute(x, order), np.transpose(x, order))


def test_where_and_masked_fill():
    c, x, y = f32(4, 5), f32(4, 5), f32(4, 5)
    np.testing.assert_array_equal(cref.where(c, x, y), np.where(c > 0, x, y))
    np.testing.assert_array_equal(cref.where(c, x, np.float32(0)), np.where(c > 0, x, 0).astype(np.float32))
    np.testing.assert_array_equal(cref.where(c, np.float32(1), np.float32(0)), (c > 0).astype(np.float32))
    x4 = f32(2, 3, 4, 4)
    mask = (RNG.random((4, 4)) > 0.5).astype(np.float32)
    for fill in (0.0, -1e9, -np.inf, np.inf):
        np.testing.assert_array_equal(cref.masked_fill(x4, mask, fill), np.where(mask > 0, np.float32(fill), x4))
    for ms in bcast_cases((2, 3, 4, 4)):
        m = (RNG.random(ms) > 0.5).astype(np.float32)
        np.testing.assert_array_equal(cref.masked_fill(x4, m, 7.0), np.where(m > 0, np.float32(7), x4))


def test_matmul_brute_force_tiny():
    x = RNG.integers(-3, 4, (3, 4)).astype(np.float32)
    y = RNG.integers(-3, 4, (4, 2)).astype(np.float32)
    want = np.zeros((3, 2), np.float32)
    for i in range(3):
        for j in range(2):
            for k in range(4):
                want[i, j] += x[i, k] * y[k, j]
    np.testing.assert_array_equal(cref.matmul(x, y), want)


@pytest.mark.parametrize("xs,ys", [((5, 7), (7, 3)), ((128, 784), (784, 64)), ((4, 5, 7), (4, 7, 3)),
                                   ((4, 5, 7), (1, 7, 3)), ((1, 5, 7), (4, 7, 3)),
                                   ((2, 3, 5, 7), (2, 3, 7, 4)), ((2, 1, 5, 7), (2, 3, 7, 4)),
                                   ((2, 3, 5, 7), (1, 1, 7, 4)), ((1, 3, 5, 7), (2, 1, 7, 4))])
def test_matmul_against_float64(xs, ys):
    x, y = f32(*xs), f32(*ys)
    want = np.matmul(x.astype(np.float64), y.astype(np.float64))
    got = cref.matmul(x, y)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4 * np.abs(want).max())


def test_matmul_transposed_operands_match_identity():
    # (A^T)^T A^T ... use an identity to catch a transposed operand: A @ I == A exactly
    a = f32(9, 6)
    np.testing.assert_array_equal(cref.matmul(a, np.eye(6, dtype=np.float32)), a)
    np.testing.assert_array_equal(cref.matmul(np.eye(9, dtype=np.float32), a), a)


def test_embedding_gather_and_scatter():
    table = f32(100, 32)
    idx = RNG.integers(0, 100, (4, 16)).astype(np.float32)
    np.testing.assert_array_equal(cref.embedding(table, idx), table[idx.astype(np.int64)])
    g = f32(4, 16, 32)
    want = np.zeros((100, 32), np.float64)
    np.add.at(want, idx.astype(np.int64).ravel(), g.reshape(-1, 32).astype(np.float64))
    np.testing.assert_allclose(cref.embedding_backward((100, 32), idx, g), want, rtol=1e-5, atol=1e-5)
    # below 2**24 the reference's float index and the integer index agree exactly
    np.testing.assert_array_equal(cref.embedding_backward((100, 32), idx, g, float_index=True),
                                  cref.embedding_backward((100, 32), idx, g))


def test_embedding_backward_float_index_breaks_above_2_24():
    # id 21846 * 768 = 16777728 > 2**24: the float expression idx*W + j cannot hit odd columns
    W, V = 768, 21850
    idx = np.array([21846.0], np.float32)
    g = np.arange(1, W + 1, dtype=np.float32).reshape(1, W)
    exact = cref.embedding_backward((V, W), idx, g)
    np.testing.assert_array_equal(exact[21846], g[0])
    literal = cref.embedding_backward((V, W), idx, g, float_index=True)
    assert not np.array_equal(literal[21846], g[0])


def test_cross_entropy_helpers():
    lsm = f32(12, 9)
    t = RNG.integers(0, 9, (12, 1)).astype(np.float32)
    np.testing.assert_array_equal(cref.ce_forward(lsm, t), lsm[np.arange(12), t[:, 0].astype(int)])
    p = lsm.copy()
    cref.ce_backward_(p, t)
    onehot = np.zeros_like(lsm)
    onehot[np.arange(12), t[:, 0].astype(int)] = 1
    np.testing.assert_array_equal(p, lsm - onehot)


def test_fills():
    np.testing.assert_array_equal(cref.arange((3, 4)), np.arange(12, dtype=np.float32).reshape(3, 4))
    np.testing.assert_array_equal(cref.full((2, 3), 1.0), np.ones((2, 3), np.float32))
    np.testing.assert_array_equal(cref.full((2, 3), 0.5), np.zeros((2, 3), np.float32))      # int(0.5) == 0
    np.testing.assert_array_equal(cref.full((2, 3), -2.7), np.full((2, 3), -2, np.float32))
    np.testing.assert_array_equal(cref.full((2, 3), 0.5, strict=False), np.full((2, 3), 0.5, np.float32))


def test_pcg32_published_vector():
    # pcg32 demo, pcg32_srandom_r(&rng, 42u, 54u): first six outputs
    want = [0xa15c02b7, 0x7b47f409, 0xba1d3330, 0x83d2f293, 0xbfa4784b, 0xcbed606e]
    np.testing.assert_array_equal(cref.pcg32_raw(6, 42, 54), np.array(want, np.uint32))
    u = cref.uniform((20000,), -0.5, 1.5, seed=42)
    assert u.min() >= -0.5 and u.max() <= 1.5
    assert abs(u.mean() - 0.5) < 0.02 and abs(u.var() - 4 / 12) < 0.02
    raw = cref.pcg32_raw(3, 42, 54).astype(np.float64) / 2 ** 32
    np.testing.assert_array_equal(cref.uniform((3,), 0.0, 1.0, seed=42), raw.astype(np.float32))
