"""GPU parity: element-wise, broadcast, select and fill kernels against the C oracle.

Tolerances are the ones the task states: bit-exact for selects/masks/fills and for
+ - * (single IEEE operations), 1e-6 relative for division and the transcendental
unary ops.  The shape matrix is the reference's (test/test_ops.py:29-75, :347-384)."""
import numpy as np
import pytest

from dlgrad_amd.buffer import Buffer
from dlgrad_amd.device import Device
from oracle import cref
from dlgrad_amd.runtime import hip
from tests.hip_util import check, dev, rel_err, require_gpu

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(11)


def f32(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


def bcast_cases(shape):
    return [tuple(1 if (m >> i) & 1 else d for i, d in enumerate(shape)) for m in range(2 ** len(shape))]


OPS = {"add": lambda a, b: a + b, "sub": lambda a, b: a - b, "mul": lambda a, b: a * b,
       "div": lambda a, b: a / b}


@pytest.mark.parametrize("op", list(OPS))
@pytest.mark.parametrize("shape", [(2, 3, 4, 5), (2, 3, 4), (784, 64), (1030,)])
def test_binary_broadcast_matrix(op, shape):
    require_gpu()
    x = f32(*shape)
    tol = 1e-6 if op == "div" else 0
    for ys in bcast_cases(shape):
        y = f32(*ys) + (3 if op == "div" else 0)
        want = cref.binary(op, x, y)
        check(OPS[op](dev(x), dev(y)).numpy(), want, tol, f"{op} {shape} {ys}")
        # smaller operand on the left: Buffer swaps, negates (sub) or inverts (div)
        if op in ("add", "mul"):
            check(OPS[op](dev(y), dev(x)).numpy(), want, tol, f"r{op} {shape} {ys}")
    check(OPS[op](dev(x), 2.5).numpy(), cref.binary(op, x, np.float32(2.5)), tol, f"{op} scalar")


def test_reversed_sub_and_div():
    require_gpu()
    x, y = f32(6, 8), f32(1, 8) + 3
    check((dev(y) - dev(x)).numpy(), cref.unary("neg", cref.binary("sub", x, y)), 0, "small-big")
    check((dev(y) / dev(x)).numpy(), cref.binary("mul", cref.unary("pow", x, -1), y), 1e-6, "small/big")
    check((3.0 - dev(x)).numpy(), np.float32(3.0) - x, 0, "scalar - x")


@pytest.mark.parametrize("shape,ys", [((4096, 4096), (4096, 4096)), ((4096, 4096), (4096, 1)),
                                      ((4096, 4096), (1, 4096)), ((16, 128, 128), (1, 128, 128)),
                                      ((16, 4, 128, 128), (16, 4, 128, 1)), ((16, 128, 128), (1, 1, 128)),
                                      ((1023, 1021), (1023, 1)), ((1023, 1021), (1, 1021))])
def test_binary_config_shapes(shape, ys):
    require_gpu()
    x, y = f32(*shape), f32(*ys) + 3
    bx, by = dev(x), dev(y)
    for op in OPS:
        check(OPS[op](bx, by).numpy(), cref.binary(op, x, y), 1e-6 if op == "div" else 0, f"{op} {shape}{ys}")


def test_device_scalar_operand_and_views():
    require_gpu()
    x = f32(33, 17)
    s = dev(np.float32(1.5).reshape(1, 1))
    check((dev(x) * s).numpy(), x * np.float32(1.5), 0, "sptr")
    # a view that starts 4 bytes into a block is not 16-byte aligned: scalar-width kernel
    base = dev(f32(1 + 33 * 17))
    view = Buffer(base.ptr + 1, (33, 17), Device.HIP)
    want = base.numpy()[1:].reshape(33, 17)
    check((view + dev(x)).numpy(), want + x, 0, "unaligned view")


def test_comparisons_and_cmp():
    require_gpu()
    x = RNG.integers(-2, 3, (37, 41)).astype(np.float32)
    y = RNG.integers(-2, 3, (37, 41)).astype(np.float32)
    check((dev(x) == dev(y)).numpy(), cref.binary("eq", x, y), 0, "eq")
    check((dev(x) > 0.0).numpy(), cref.binary("gt", x, np.float32(0)), 0, "gt")
    check((dev(x) >= 1.0).numpy(), cref.binary("gte", x, np.float32(1)), 0, "gte")
    H, W = 128, 128
    cols, rows = np.arange(W, dtype=np.float32).reshape(1, W), np.arange(H, dtype=np.float32).reshape(H, 1)
    check((dev(cols) <= dev(rows)).numpy(), cref.cmp_le(cols, rows, (H, W)), 0, "cmp<=")


@pytest.mark.parametrize("n", [1, 5, 1024, 4097, 1 << 20])
def test_unary(n):
    require_gpu()
    x = f32(n)
    pos = np.abs(x) + np.float32(1e-3)
    check((-dev(x)).numpy(), cref.unary("neg", x), 0, "neg")
    check(dev(x).exp().numpy(), cref.unary("exp", x), 1e-6, "exp")
    check(dev(pos).log().numpy(), cref.unary("log", pos), 1e-6, "log")
    check(dev(pos).sqrt().numpy(), cref.unary("sqrt", pos), 1e-6, "sqrt")
    check(dev(pos).rsqrt().numpy(), cref.unary("rsqrt", pos), 1e-6, "rsqrt")
    for p in (2.0, 3.0, -1.0, 0.0):
        check((dev(pos) ** p).numpy(), cref.unary("pow", pos, p), 1e-6, f"pow {p}")
    check(dev(x).clamp(-0.5, 0.25).numpy(), cref.clamp(x, -0.5, 0.25), 0, "clamp")
    check(dev(x).clamp(min=0).numpy(), cref.clamp(x, 0, None), 0, "clamp min")
    check(dev(x).clamp(max=0.1).numpy(), cref.clamp(x, None, 0.1), 0, "clamp max")


def test_exp_of_minus_inf_and_log_edge_values():
    require_gpu()
    x = np.array([-np.inf, -100.0, 0.0, 88.0, 1e-30], np.float32)
    check(dev(x).exp().numpy(), np.exp(x.astype(np.float64)).astype(np.float32), 1e-6, "exp edge")


def test_special_values_follow_the_reference_source_read_as_ieee():
    """NaN, the infinities, signed zeros, denormals and the extremes through the element-wise ops, the max reductions and
    argmax.  The reference builds its kernels with -ffast-math (cpu.py:30-41), which leaves NaN and infinite operands to
    the compiler: the C restatement built with the same flags answers NaN to inf / 0 and to rsqrt(inf), and lets a NaN
    decide a max or an argmax.  So the oracle here is the reference's *source* read under IEEE rules, evaluated with
    numpy: x / y, 1 / sqrt(x), cond > 0 ? x : y (relu is where(x, x, 0), buffer.py:338-342), and the scans
    `if (v > best)` from (-FLT_MAX, 0), which a NaN never enters (cpu_kernel.py:68-148, :459-517)."""
    require_gpu()
    vals = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1e-45, -1e-45, 1e-38, 3.4e38, -3.4e38, 1.0, -1.0, 2.5, -2.5, 88.8, -104.0], np.float32)
    a, b = np.repeat(vals, len(vals)), np.tile(vals, len(vals))
    ad, bd = dev(a), dev(b)

    def agree(got, want, what, tol=0.0):
        if hip.COMPILE_ONLY:
            return
        want = np.asarray(want, np.float32)
        same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
        if tol:
            fin = np.isfinite(got) & np.isfinite(want)
            same |= fin & (np.abs(got.astype(np.float64) - want) <= tol * np.abs(want) + 1.5e-45)
        bad = np.flatnonzero(~same)
        assert not bad.size, f"{what}: " + "; ".join(f"({a[i]}, {b[i]}) -> {got[i]}, expected {want[i]}" for i in bad[:5])
    with np.errstate(all="ignore"):
        agree((ad + bd).numpy(), a + b, "add")
        agree((ad - bd).numpy(), a - b, "sub")
        agree((ad * bd).numpy(), a * b, "mul")
        agree((ad / bd).numpy(), a / b, "div", 1e-6)
        agree((ad > bd).numpy(), (a > b).astype(np.float32), "greater")
        agree((ad == bd).numpy(), (a == b).astype(np.float32), "equal")
        agree(ad.where(ad, bd).numpy(), np.where(a > 0, a, b), "where")
        agree(ad.relu().numpy(), np.where(a > 0, a, np.float32(0)), "relu")
        agree((-ad).numpy(), -a, "neg")
        agree(ad.exp().numpy(), np.exp(a.astype(np.float64)), "exp", 1e-6)
        agree(ad.log().numpy(), np.log(a.astype(np.float64)), "log", 1e-6)
        agree(ad.sqrt().numpy(), np.sqrt(a), "sqrt", 1e-6)
        agree(ad.rsqrt().numpy(), 1.0 / np.sqrt(a.astype(np.float64)), "rsqrt", 1e-6)
    rows = np.stack([np.roll(vals, s) for s in range(len(vals))] + [np.where(np.isnan(np.roll(vals, s)), 1.0, np.roll(vals, s)) for s in range(4)]).astype(np.float32)

    def scan(v):                                   # the reference's loop: (best, index) from (-FLT_MAX, 0), strict '>'
        best, at = -np.finfo(np.float32).max, 0
        for i, x in enumerate(v):
            if x > best:
                best, at = x, i
        return best, at
    rd = dev(rows)
    for axis in (0, 1):
        lines = rows.T if axis == 0 else rows
        want = [scan(v) for v in lines]
        got_max, got_arg = rd.max(axis).numpy().ravel(), rd.argmax(axis).numpy().ravel()
        if not hip.COMPILE_ONLY:
            np.testing.assert_array_equal(got_max, np.array([w[0] for w in want], np.float32), err_msg=f"max over axis {axis}")
            np.testing.assert_array_equal(got_arg, np.array([w[1] for w in want], np.float32), err_msg=f"argmax over axis {axis}")
        got_sum = rd.sum(axis).numpy().ravel()
        with np.errstate(all="ignore"):
            ref = lines.astype(np.float64).sum(1)
        if not hip.COMPILE_ONLY:
            assert (np.isnan(got_sum) == np.isnan(ref)).all() and (got_sum[np.isinf(ref)] == ref[np.isinf(ref)]).all(), f"sum over axis {axis}"


def test_where_relu_masked_fill():
    require_gpu()
    c, x, y = f32(64, 50), f32(64, 50), f32(64, 50)
    check(dev(c).where(dev(x), dev(y)).numpy(), cref.where(c, x, y), 0, "where ttt")
    check(dev(c).where(dev(x), 0.0).numpy(), cref.where(c, x, np.float32(0)), 0, "where tts")
    check(dev(c).where(1.0, 0.0).numpy(), cref.where(c, np.float32(1), np.float32(0)), 0, "where tss")
    check(dev(x).relu().numpy(), cref.where(x, x, np.float32(0)), 0, "relu")
    check(dev(x).leaky_relu(0.01).numpy(), cref.where(x, x, x * np.float32(0.01)), 0, "leaky")
    x4 = f32(2, 3, 8, 8)
    for ms in bcast_cases((2, 3, 8, 8)) + [(8, 8), (8,)]:
        m = (RNG.random(ms) > 0.5).astype(np.float32)
        for fill in (7.0, -np.inf):
            check(Buffer.masked_fill(dev(x4), dev(m), fill).numpy(), cref.masked_fill(x4, m, fill), 0,
                  f"masked_fill {ms} {fill}")
    att = f32(16, 4, 128, 128)
    mask = 1 - np.tril(np.ones((128, 128), np.float32))
    check(Buffer.masked_fill(dev(att), dev(mask), float("-inf")).numpy(),
          cref.masked_fill(att, mask, -np.inf), 0, "causal mask")


def test_fills():
    require_gpu()
    check(Buffer.arange((128, 1), Device.HIP).numpy(), cref.arange((128, 1)), 0, "arange")
    check(Buffer.full((3, 5), 1.0, Device.HIP).numpy(), cref.full((3, 5), 1.0), 0, "full 1")
    from dlgrad_amd.helpers import STRICT_REFERENCE
    want_half = cref.full((3, 5), 0.5) if STRICT_REFERENCE else np.full((3, 5), 0.5, np.float32)    # (the reference's int cast is what strictness keeps)
    check(Buffer.full((3, 5), 0.5, Device.HIP).numpy(), want_half, 0, "full int-truncated")
    check(Buffer.full((1027,), -3.0, Device.HIP).numpy(), cref.full((1027,), -3.0), 0, "full tail")
    u = Buffer.uniform((100000,), Device.HIP, "float32", low=-2.0, high=2.0).numpy()
    if u.any():
        assert u.min() >= -2 and u.max() < 2 and abs(u.mean()) < 0.05


@pytest.mark.parametrize("n", [1, 6, 255, 256, 257, 100003, 4096 * 256 + 77, 3_000_001])
def test_uniform_is_the_sequential_pcg32_stream(n):
    """Element i is the i-th output of PCG32 (seed, stream), however many threads shared the
    work: bit-exact in the [0, 1) form, where no arithmetic follows the conversion; the affine
    form may differ from the oracle by the rounding of one fused multiply-add (the reference's
    -ffast-math leaves that contraction to its compiler)."""
    require_gpu()
    import dlgrad_amd
    from dlgrad_amd.runtime.hip import HIP
    dlgrad_amd.manual_seed(42)
    HIP._stream = 54
    got = Buffer.uniform((n,), Device.HIP, "float32").numpy()
    assert HIP._stream == 55
    check(got, cref.uniform((n,), 0.0, 1.0, seed=42, seq=54), 0, f"U[0,1) n={n}")
    if n >= 6 and not hip.COMPILE_ONLY:       # the published pcg32 demo vector (seed 42, sequence 54)
        want = np.array([0xa15c02b7, 0x7b47f409, 0xba1d3330, 0x83d2f293, 0xbfa4784b, 0xcbed606e], np.float64)
        np.testing.assert_array_equal(got[:6], (want / 2 ** 32).astype(np.float32))
    HIP._stream = 7
    got = Buffer.uniform((n,), Device.HIP, "float32", low=-0.0357, high=0.0357).numpy()
    want = cref.uniform((n,), -0.0357, 0.0357, seed=42, seq=7)
    if not hip.COMPILE_ONLY:
        assert np.abs(got - want).max() <= np.spacing(np.float32(0.0357))
        assert got.min() >= np.float32(-0.0357) and got.max() <= np.float32(0.0357)


def test_seeded_layers_start_equal_on_both_devices():
    """manual_seed + the per-call streams give the hip device and the oracle's cpu device the
    same initial weights."""
    require_gpu()
    import dlgrad_amd
    import oracle.cpu_runtime as ocpu
    from dlgrad_amd import nn
    dlgrad_amd.manual_seed(5)
    ocpu.CPU.manual_seed(5)
    a, b = nn.Linear(33, 17, device="hip"), nn.Linear(33, 17, device="cpu")
    if not hip.COMPILE_ONLY:
        assert np.abs(a.weight.numpy() - b.weight.numpy()).max() <= np.spacing(np.float32(33 ** -0.5))
        assert np.abs(a.bias.numpy() - b.bias.numpy()).max() <= np.spacing(np.float32(33 ** -0.5))
        assert not np.array_equal(a.weight.numpy().ravel()[:17], a.bias.numpy().ravel())     # different streams


def test_dropout_mask_comes_from_the_seeded_stream():
    """dropout(p) keeps x / (1 - p) where the stream's U[0,1) value is >= p and zeroes the rest
    (ops.py:442-462); the gradient passes through the same mask."""
    require_gpu()
    import dlgrad_amd
    from dlgrad_amd import Tensor
    x = f32(64, 100)
    dlgrad_amd.manual_seed(9)
    t = Tensor(x, device="hip", requires_grad=True)
    y = t.dropout(0.3)
    y.sum().backward()
    if hip.COMPILE_ONLY:
        return
    keep = cref.uniform((64, 100), 0.0, 1.0, seed=9, seq=0) >= np.float32(0.3)
    scale = np.float32(1.0 / (1.0 - 0.3))
    check(y.numpy(), np.where(keep, x, np.float32(0)) * scale, 0, "dropout forward")
    check(t.grad.numpy(), np.where(keep, np.float32(1), np.float32(0)) * scale, 0, "dropout backward")
    assert 0.6 < keep.mean() < 0.8


# ---- the streaming ("nt") forms -------------------------------------------------------------------
# From NT_STORE_MIN_ELEMENTS (2^25) elements on, the launcher picks kernel variants that read
# and write with nontemporal accesses and walk one 16-byte item per thread.  They are the
# variants the C2 benchmark times at 16384 x 8192, so they are compared with the oracle twice:
# every variant at a small size (threshold lowered), and the suite's shapes at full size.

@pytest.fixture
def streaming_everywhere(monkeypatch):
    """Lowers the streaming threshold so that tensors of a few thousand elements take the nt
    kernels; launch plans made under the other threshold are set aside for the test."""
    monkeypatch.setattr(hip, "NT_STORE_MIN_ELEMENTS", 1024)
    monkeypatch.setattr(hip, "_map_plans", {})
    yield


def test_streaming_map_variants_match_the_oracle(streaming_everywhere):
    require_gpu()
    R, C = 96, 520                                                 # 49920 elements: a ragged last block
    x, same = f32(R, C), f32(R, C) + 3
    col, row = f32(R, 1) + 3, f32(1, C) + 3
    one = dev((f32(1, 1) + 3))
    bx = dev(x)
    n0 = len(hip.requested_kernels)
    for op in OPS:
        tol = 1e-6 if op == "div" else 0
        for name, y in (("same", same), ("(R,1)", col), ("(1,C)", row)):
            check(OPS[op](bx, dev(y)).numpy(), cref.binary(op, x, y), tol, f"nt {op} {name}")
        check(OPS[op](bx, 1.5).numpy(), cref.binary(op, x, np.float32(1.5)), tol, f"nt {op} scalar")
        check(OPS[op](bx, one).numpy(), cref.binary(op, x, one.numpy()), tol, f"nt {op} device scalar")
    pos = np.abs(x) + np.float32(1e-3)
    check(bx.exp().numpy(), cref.unary("exp", x), 1e-6, "nt exp")
    check(dev(pos).log().numpy(), cref.unary("log", pos), 1e-6, "nt log")
    check(dev(pos).sqrt().numpy(), cref.unary("sqrt", pos), 1e-6, "nt sqrt")
    check(dev(pos).rsqrt().numpy(), cref.unary("rsqrt", pos), 1e-6, "nt rsqrt")
    check((-bx).numpy(), cref.unary("neg", x), 0, "nt neg")
    check((dev(pos) ** 3.0).numpy(), cref.unary("pow", pos, 3.0), 1e-6, "nt pow")
    check(bx.clamp(-0.5, 0.25).numpy(), cref.clamp(x, -0.5, 0.25), 0, "nt clamp")
    check(bx.relu().numpy(), cref.where(x, x, np.float32(0)), 0, "nt relu")
    check(bx.where(dev(same), dev(x)).numpy(), cref.where(x, same, x), 0, "nt where, three tensors")
    check((bx > 0.0).numpy(), cref.binary("gt", x, np.float32(0)), 0, "nt gt")
    m = (RNG.random((1, C)) > 0.5).astype(np.float32)
    check(Buffer.masked_fill(bx, dev(m), float("-inf")).numpy(), cref.masked_fill(x, m, -np.inf), 0, "nt masked_fill")
    check(Buffer.full((R, C), 2.0, Device.HIP).numpy(), cref.full((R, C), 2.0), 0, "nt full")
    names = {hip_kernel_name(g, p) for g, p in hip.requested_kernels}
    if len(hip.requested_kernels) > n0 or not hip.COMPILE_ONLY:
        assert any(n.endswith("u1nt") for n in names), "the streaming variants were not selected"


def hip_kernel_name(gen_name: str, params: tuple) -> str:
    from dlgrad_amd.codegen import hip_kernel as K
    return getattr(K, gen_name)(*params)[1]


def test_streaming_reduce_argmax_permute_softmax_variants_match_the_oracle(streaming_everywhere):
    require_gpu()
    x = f32(192, 2304)                                             # rows long enough for the block-per-row forms
    bx = dev(x)
    f64 = x.astype(np.float64)
    def close_sum(got, want, what):          # sums of N(0,1) values cancel: measured against the largest |sum|
        if not hip.COMPILE_ONLY:
            assert got.shape == want.shape and np.abs(got - want).max() <= 1e-5 * np.abs(want).max() + 1e-4, what
    for dim in (0, 1, None):
        args = () if dim is None else (dim,)
        check(bx.max(*args).numpy(), np.asarray(x.max(*args)), 0, f"nt max {dim}")
        close_sum(bx.sum(*args).numpy(), np.asarray(f64.sum(*args)), f"nt sum {dim}")
    ones = np.ones((192, 2304), np.float32)
    check(dev(ones).sum(0).numpy(), ones.sum(0), 0, "nt sum axis 0 of ones")
    check(dev(ones).sum(1).numpy(), ones.sum(1), 0, "nt sum axis 1 of ones")
    check(dev(ones).sum().numpy(), np.asarray(ones.sum()), 0, "nt sum of ones")
    planted = x.copy()
    planted[:, 7] = planted[:, 900] = 9.0                          # ties: the first maximum wins
    planted[5, :] = -np.inf
    bp = dev(planted)
    check(bp.argmax(1).numpy(), cref.argmax(planted, 1).reshape(-1, 1), 0, "nt argmax rows")
    tall = f32(4096, 256)
    tall[100] = tall[3000] = 9.0
    check(dev(tall).argmax(0).numpy(), cref.argmax(tall, 0).reshape(1, -1), 0, "nt argmax columns")
    check(bx.permute((1, 0)).numpy(), cref.permute(x, (1, 0)), 0, "nt transpose")
    sq = f32(1024, 2048)                                           # a 2 KiB-multiple pitch: the diagonal 128 x 128 tiles
    check(dev(sq).permute((1, 0)).numpy(), cref.permute(sq, (1, 0)), 0, "nt transpose, diagonal tiles")
    h = f32(4, 64, 6, 32)
    check(dev(h).permute((0, 2, 1, 3)).numpy(), cref.permute(h, (0, 2, 1, 3)), 0, "nt head permute")
    rows = f32(64, 1024)
    e = np.exp(rows.astype(np.float64) - rows.astype(np.float64).max(1, keepdims=True))
    want = e / e.sum(1, keepdims=True)
    got = dev(rows).softmax(1)
    check(got.numpy(), want, 2e-6, "nt softmax")
    g = f32(64, 1024)
    y64 = want
    dwant = y64 * (g - (g * y64).sum(1, keepdims=True))
    dgot = got.softmax_bwd(dev(g)).numpy()
    if not hip.COMPILE_ONLY:                                       # cancellation: measured against the largest entry
        assert np.abs(dgot - dwant).max() <= 2e-6 * np.abs(dwant).max(), "nt softmax backward"
    mask = np.triu(np.ones((64, 1024), np.float32), 1)
    z = np.where(mask > 0, -np.inf, rows.astype(np.float64) * 0.125)
    ez = np.exp(z - z.max(1, keepdims=True))
    check(dev(rows).masked_softmax(dev(mask), 0.125).numpy(), ez / ez.sum(1, keepdims=True), 2e-6, "nt masked softmax")


@pytest.mark.parametrize("case", ["add_same", "sub_rowvec", "mul_colvec", "div_scalar", "exp", "relu", "log", "sqrt"])
def test_c2_suite_at_16384x8192_matches_the_oracle(case):
    """The benchmark's own size: 134 M elements per tensor, the streaming kernels as the launcher
    picks them with its default threshold."""
    require_gpu()
    R, C = 16384, 8192
    rng = np.random.default_rng(2)
    a = rng.standard_normal((R, C), dtype=np.float32)
    da = dev(a)
    if case == "add_same":
        b = rng.standard_normal((R, C), dtype=np.float32)
        got, want, tol = (da + dev(b)).numpy(), (lambda: cref.binary("add", a, b)), 0
    elif case == "sub_rowvec":
        v = rng.standard_normal((R, 1), dtype=np.float32)
        got, want, tol = (da - dev(v)).numpy(), (lambda: cref.binary("sub", a, v)), 0
    elif case == "mul_colvec":
        v = rng.standard_normal((1, C), dtype=np.float32)
        got, want, tol = (da * dev(v)).numpy(), (lambda: cref.binary("mul", a, v)), 0
    elif case == "div_scalar":
        got, want, tol = (da / 1.5).numpy(), (lambda: cref.binary("div", a, np.float32(1.5))), 1e-6
    elif case == "exp":
        got, want, tol = da.exp().numpy(), (lambda: cref.unary("exp", a)), 1e-6
    elif case == "relu":
        got, want, tol = da.relu().numpy(), (lambda: cref.where(a, a, np.float32(0))), 0
    else:
        pos = np.abs(a) + np.float32(1e-3)
        got, want, tol = getattr(dev(pos), case)().numpy(), (lambda: cref.unary(case, pos)), 1e-6
    if hip.COMPILE_ONLY:                                        # the kernel-recording run: no result to compare, so no oracle pass either
        return
    want = want()
    assert got.shape == want.shape
    if tol == 0:
        assert np.array_equal(got, want), case
    else:
        g, w = got.reshape(-1), want.reshape(-1)                # NaN-strict (rel_err), a slab at a time to bound float64 temporaries
        step = 1 << 24
        worst = max(rel_err(g[i:i + step], w[i:i + step]) for i in range(0, g.size, step))
        assert worst <= tol, (case, worst)
