"""GPU parity: element-wise map / map2 / map3 through the C ABI against the CPU oracle on identical seeded inputs.
Bar: bit-exact for integer/bool work and for the exactly rounded fp ops (+ - * / sqrt abs neg min max rounding);
1e-6 relative for transcendentals (the oracle is double libm rounded to T; the kernels use correctly-implemented
single-precision routines, no fast-math)."""
import numpy as np
import pytest

from util import both, assert_exact, assert_rel

pytestmark = pytest.mark.gpu

NUM = [np.uint8, np.int8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64, np.float32, np.float64]


def rand(rng, dt, shape, lo=-50, hi=50):
    dt = np.dtype(dt)
    if dt.kind == "f":
        return (rng.random(shape) * (hi - lo) + lo).astype(dt)
    if dt.kind == "u":
        return rng.integers(0, min(hi * 2, np.iinfo(dt).max), size=shape).astype(dt)
    if dt.kind == "b":
        return rng.random(shape) < 0.5
    return rng.integers(max(lo, np.iinfo(dt).min), min(hi, np.iinfo(dt).max), size=shape).astype(dt)


@pytest.mark.parametrize("dt", NUM)
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "mod", "max", "min"])
def test_binary_exact(H, G, rng, dt, op):
    a = rand(rng, dt, (37, 129))
    b = rand(rng, dt, (37, 129))
    if op in ("div", "mod"):
        b[b == 0] = 3
    f = {"add": lambda x, y: x + y, "sub": lambda x, y: x - y, "mul": lambda x, y: x * y, "div": lambda x, y: x / y,
         "mod": lambda x, y: x % y, "max": lambda x, y: type(x).maxElemwise(x, y), "min": lambda x, y: type(x).minElemwise(x, y)}[op]
    ref, got = both(H, G, f, a, b)
    assert_exact(ref, got)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("fn,lo,hi", [("log", 0.01, 50), ("log10", 0.01, 50), ("exp", -20, 20), ("sin", -20, 20), ("cos", -20, 20),
                                      ("tan", -1.5, 1.5), ("asin", -1, 1), ("acos", -1, 1), ("atan", -50, 50), ("sinh", -10, 10),
                                      ("cosh", -10, 10), ("tanh", -5, 5)])
def test_transcendental_rel(H, G, rng, dt, fn, lo, hi):
    a = rand(rng, dt, (1000, 65), lo, hi)
    ref, got = both(H, G, lambda x: getattr(x, fn)(), a)
    assert_rel(ref, got, 1e-6)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("fn", ["sqrt", "ceiling", "floor", "round", "truncate", "abs", "sgn", "__neg__", "__pos__"])
def test_unary_exact_fp(H, G, rng, dt, fn):
    a = rand(rng, dt, (513, 33), 0 if fn == "sqrt" else -50, 50)
    a.flat[:8] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.0, -0.0] if fn != "sqrt" else [0.5, 1.5, 2.5, 0.25, 4, 9, 0.0, 2.0]
    ref, got = both(H, G, lambda x: getattr(x, fn)(), a)
    assert_exact(ref, got)


def test_special_values_fp(H, G):
    for dt in (np.float32, np.float64):
        a = np.array([np.inf, -np.inf, np.nan, 0.0, -0.0, 1.0, -1.0, 1e-40, 3e38], dtype=dt)
        for fn in ["tanh", "exp", "atan", "sqrt", "abs", "sgn", "floor", "round"]:
            with np.errstate(all="ignore"):
                ref, got = both(H, G, lambda x: getattr(x, fn)(), a)
            assert_rel(ref, got, 1e-6)
        ref, got = both(H, G, lambda x: x.isFinite(), a)
        assert_exact(ref, got)


@pytest.mark.parametrize("dt", [np.int8, np.int16, np.int32, np.int64])
def test_unary_int(H, G, rng, dt):
    a = rand(rng, dt, (100, 17))
    for fn in ["__neg__", "abs", "__pos__"] + (["sgn"] if dt != np.int8 else []):
        ref, got = both(H, G, lambda x: getattr(x, fn)(), a)
        assert_exact(ref, got)


def test_unsupported_raise(G, rng):
    a = G.ofNumpy(rand(rng, np.uint32, (8,)))
    with pytest.raises(NotImplementedError):
        -a
    with pytest.raises(NotImplementedError):
        G.ofNumpy(rand(rng, np.int32, (8,))).tanh()
    with pytest.raises(NotImplementedError):
        G.ofNumpy(rand(rng, np.int32, (8,))) ** G.ofNumpy(rand(rng, np.int32, (8,)))


def test_integer_wraparound(H, G):
    a = np.array([2 ** 31 - 1, -2 ** 31, 123456789, -5], dtype=np.int32)
    b = np.array([1, -1, 987654321, 3], dtype=np.int32)
    for f in (lambda x, y: x + y, lambda x, y: x - y, lambda x, y: x * y):
        ref, got = both(H, G, f, a, b)
        assert_exact(ref, got)
    # truncation toward zero
    ref, got = both(H, G, lambda x, y: x / y, np.array([-7, 7, -7, 7], np.int32), np.array([2, -2, -2, 2], np.int32))
    assert_exact(ref, got)
    assert got.tolist() == [-3, -3, 3, 3]
    ref, got = both(H, G, lambda x, y: x % y, np.array([-7, 7, -7, 7], np.int32), np.array([2, -2, -2, 2], np.int32))
    assert got.tolist() == [-1, 1, -1, 1]


@pytest.mark.parametrize("dt", [np.int8, np.int16, np.int32, np.int64, np.uint16, np.uint64])
def test_integer_division_corner_cases(H, G, dt):
    """A zero divisor gives 0.  MinValue / -1: 0 for int32 / int64 (the quotient does not exist); the narrower types divide as
    int32 and wrap when the quotient is stored, so MinValue comes back."""
    info = np.iinfo(dt)
    a = np.array([info.min, info.max, 7, info.min, 0], dtype=dt)
    b = np.array([0, 0, 0, info.max if info.min == 0 else -1, 0], dtype=dt)
    ref, got = both(H, G, lambda x, y: x / y, a, b)
    assert_exact(ref, got)
    narrow_signed = info.min < 0 and np.dtype(dt).itemsize < 4
    assert got.tolist() == [0, 0, 0, info.min if narrow_signed else 0, 0]
    ref, got = both(H, G, lambda x, y: x % y, a, b)
    assert_exact(ref, got)
    assert got.tolist() == [0, 0, 0, 0, 0]


@pytest.mark.parametrize("dt", [np.bool_] + NUM)
def test_compare(H, G, rng, dt):
    a = rand(rng, dt, (63, 70), -3, 3)
    b = rand(rng, dt, (63, 70), -3, 3)
    for f in (lambda x, y: x == y, lambda x, y: x != y, lambda x, y: x < y, lambda x, y: x <= y, lambda x, y: x > y, lambda x, y: x >= y):
        ref, got = both(H, G, f, a, b)
        assert_exact(ref, got)


def test_logic(H, G, rng):
    a = rand(rng, np.bool_, (1000,))
    b = rand(rng, np.bool_, (1000,))
    for f in (lambda x, y: x & y, lambda x, y: x | y, lambda x, y: x ^ y, lambda x, y: ~x):
        ref, got = both(H, G, f, a, b)
        assert_exact(ref, got)


@pytest.mark.parametrize("dt", [np.bool_, np.int8, np.uint16, np.int32, np.float32, np.int64, np.float64])
def test_if_then_else(H, G, rng, dt):
    c = rand(rng, np.bool_, (33, 65))
    a = rand(rng, dt, (33, 65))
    b = rand(rng, dt, (33, 65))
    ref, got = both(H, G, lambda c, a, b: type(a).ifThenElse(c, a, b), c, a, b)
    assert_exact(ref, got)
    assert_exact(np.where(c, a, b), got)


def test_scalar_broadcast_and_power(H, G, rng):
    a = rand(rng, np.float32, (4097,), 0.1, 5)
    ref, got = both(H, G, lambda x: x * 2.5 + 1.0, a)
    assert_exact(ref, got)
    ref, got = both(H, G, lambda x: x ** 1.7, a)
    assert_rel(ref, got, 1e-6)
    ai = rand(rng, np.int32, (100000,), -1000, 1000)
    ref, got = both(H, G, lambda x: x > 0, ai)
    assert_exact(ref, got)
    assert_exact(ai > 0, got)


@pytest.mark.parametrize("dt", [np.float32, np.float64, np.int32, np.uint8, np.int16])
def test_strided_and_broadcast_views(H, G, rng, dt):
    x = rand(rng, dt, (6, 20, 70))
    v = rand(rng, dt, (70,))
    w = rand(rng, dt, (20, 1))

    # permuted view + broadcast vector, as the frontend builds them
    def f(x, v, w):
        xp = x.permuteAxes([2, 0, 1])          # shape [20, 70, 6]
        return xp + v[None, :, None] + w[:, :, None]
    ref, got = both(H, G, f, x, v, w)
    assert_exact(ref, got)
    exp = np.transpose(x, (1, 2, 0)) + v[None, :, None] + w[:, :, None]
    assert_exact(exp.astype(dt), got)

    # slices with offsets, transposes, reversed axes, copies into non-contiguous targets
    def g(x, v, w):
        s = x[1:5, 3:17, 5:64]
        return (s.T.reverseAxis(0) - s.T).Copy()
    ref, got = both(H, G, g, x, v, w)
    assert_exact(ref, got)

    def h(x, v, w):
        t = type(x).new([70, 20], x.Dev, x.DataType).T     # column-major target of shape [20, 70]
        t.FillAdd(x[2], x[3])
        return t
    ref, got = both(H, G, h, x, v, w)
    assert_exact(ref, got)


@pytest.mark.parametrize("dt", [np.float32, np.float64, np.int32, np.uint8, np.int16, np.int64])
def test_misaligned_ragged_and_strided_rows(H, G, rng, dt):
    """Row-wise calls that the aligned vector kernels cannot take: differences of shifted views (every operand starts at another
    element), odd row lengths, a target that is itself a shifted view, a source strided along the rows, a row-broadcast and a
    column-broadcast operand beside them; NumPy is the checker, the oracle device the second one."""
    x = rand(rng, dt, (37, 1031))
    y = rand(rng, dt, (37, 1031))
    v = rand(rng, dt, (1031,))
    tx, ty, tv = G.ofNumpy(x), G.ofNumpy(y), G.ofNumpy(v)
    assert_exact(x[:, 1:] - x[:, :-1], G.toNumpy(tx[:, 1:] - tx[:, :1030]))               # row length 1030, one operand misaligned
    assert_exact(x[:, 3:1027] - y[:, 5:1029], G.toNumpy(tx[:, 3:1027] - ty[:, 5:1029]))  # whole vectors per row, both misaligned
    assert_exact(x[:, 2:] - v[None, 2:], G.toNumpy(tx[:, 2:] - tv[None, 2:]))
    assert_exact(x[:, 7:900] - y[:, 0:1][:, :].repeat(893, axis=1), G.toNumpy(tx[:, 7:900] - ty[:, 0:1].broadcastTo([37, 893])))
    assert_exact(x[1:, 1:] > y[:-1, :-1], G.toNumpy(tx[1:, 1:] > ty[:36, :1030]))
    # 1-d: the finite difference of a long vector
    z = rand(rng, dt, (100003,))
    tz = G.ofNumpy(z)
    assert_exact(z[1:] - z[:-1], G.toNumpy(tz[1:] - tz[:100002]))
    # a target that starts at an odd element and whose rows are not whole vectors
    out = G.zeros([37, 1031], dt)
    out[:, 1:].FillSubtract(tx[:, 1:], ty[:, :1030])
    want = np.zeros_like(x)
    want[:, 1:] = x[:, 1:] - y[:, :-1]
    assert_exact(want, G.toNumpy(out))
    # a source strided along the rows (a plane of a 3-d tensor) against a contiguous one
    c = rand(rng, dt, (29, 515, 3))
    d = rand(rng, dt, (29, 515))
    tc, td = G.ofNumpy(c), G.ofNumpy(d)
    assert_exact(c[:, :, 1] - d, G.toNumpy(tc[:, :, 1] - td))
    assert_exact(d[:, ::-1] - c[:, :, 2], G.toNumpy(td.reverseAxis(1) - tc[:, :, 2]))
    # transposing calls on views that start at odd elements and have odd row pitches (whole vectors per row all the same)
    m = rand(rng, dt, (200, 301))
    n = rand(rng, dt, (260, 131))
    tm, tn = G.ofNumpy(m), G.ofNumpy(n)
    sm, sn = m[1:129, 3:259], n[2:258, 1:129]
    assert_exact(np.ascontiguousarray(sm.T), G.toNumpy(tm[1:129, 3:259].T.Copy()))
    assert_exact(sm.T - sn, G.toNumpy(tm[1:129, 3:259].T - tn[2:258, 1:129]))
    assert_exact(sn - sm.T, G.toNumpy(tn[2:258, 1:129] - tm[1:129, 3:259].T))
    outv = G.zeros([260, 131], dt)
    outv[2:258, 1:129].FillSubtract(tm[1:129, 3:259].T, tn[2:258, 1:129])
    wantv = np.zeros_like(n)
    wantv[2:258, 1:129] = sm.T - sn
    assert_exact(wantv, G.toNumpy(outv))
    # the oracle device on the same views
    ref, got = both(H, G, lambda a, b: (a[:, 1:] - b[:, :1030], a[2:, 5:] + b[:35, :1026]), x, y)
    assert_exact(ref[0], got[0])
    assert_exact(ref[1], got[1])


def test_large_transpose_copy_and_add(H, G, rng):
    x = rng.standard_normal((16, 96, 200)).astype(np.float32)
    v = rng.random(200).astype(np.float32)

    def f(x, v):
        xp = x.permuteAxes([2, 0, 1])              # [96, 200, 16], strides [200, 1, 19200]
        return xp + v[None, :, None], xp.Copy()
    (r1, r2), (g1, g2) = both(H, G, f, x, v)
    assert_exact(r1, g1)
    assert_exact(r2, g2)
    assert_exact(np.transpose(x, (1, 2, 0)).copy(), g2)
    # fp64 uses the 32x32 tile variant
    xd = x.astype(np.float64)
    ref, got = both(H, G, lambda x: x.permuteAxes([2, 0, 1]).Copy(), xd)
    assert_exact(ref, got)


def test_in_place(H, G):
    # the documentation's f3.FillMultiply f3 e example, Guide-Operations.md:103-115
    def f(f3, d, e):
        f3.FillMultiply(d, e)
        f3.FillMultiply(f3, e)
        return f3
    ref, got = both(H, G, f, np.array([-1.0, -1.0, 29.0, 40.0]), np.arange(4.0), 10.0 * np.arange(4.0))
    assert_exact(ref, got)
    assert got.tolist() == [0.0, 100.0, 800.0, 2700.0]


@pytest.mark.parametrize("src", [np.bool_] + NUM)
@pytest.mark.parametrize("dst", [np.bool_] + NUM)
def test_convert(H, G, rng, src, dst):
    a = rand(rng, src, (257,), 0, 100)
    ref, got = both(H, G, lambda x: x.convert(dst), a)
    assert_exact(ref, got)
    if np.dtype(dst) != np.bool_:
        assert_exact(a.astype(dst), got)


@pytest.mark.parametrize("src", [np.int16, np.uint16, np.int32, np.int64, np.uint64])
def test_convert_between_integers_keeps_the_low_bits(H, G, rng, src):
    info = np.iinfo(src)
    a = rng.integers(info.min, info.max, size=5000, dtype=src, endpoint=True)
    a[:4] = [info.min, info.max, 0, info.max // 2 + 1]
    for dst in (np.int8, np.uint8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64):
        ref, got = both(H, G, lambda x: x.convert(dst), a)
        assert_exact(ref, got)
        assert_exact(a.astype(dst), got)            # NumPy's integer casts wrap as well


def test_convert_of_floats_outside_the_integer_range(H, G):
    """NaN, infinities and floats that do not fit the integer target: the device follows the same stated rule as the oracle (a
    plain cast would saturate on the GPU), checked against the hand-worked vectors and, in single precision, against the oracle."""
    import convert_cases as cc
    x = np.array(cc.INPUTS, dtype=np.float64)
    for dst in cc.EXPECTED:
        got = G.toNumpy(G.ofNumpy(x).convert(dst))
        assert got.dtype == np.dtype(dst)
        assert np.array_equal(got, cc.expected(dst)), (dst, got, cc.expected(dst))
        with np.errstate(all="ignore"):
            x32 = np.concatenate([x.astype(np.float32), np.float32([3e9, -3e9, 1.5e19, 7e18, -7e18, 2.5, -2.5])])
        ref, dev = both(H, G, lambda t: t.convert(dst), x32)
        assert_exact(ref, dev)


def test_fill_and_counting(H, G):
    for dt in NUM:
        ref, got = both(H, G, lambda x: type(x).filled([5, 7], 3, x.Dev, x.DataType), np.zeros(1, dt))
        assert_exact(ref, got)
        ref, got = both(H, G, lambda x: type(x).counting(1000, x.Dev, x.DataType), np.zeros(1, dt))
        assert_exact(ref, got)
    got = G.toNumpy(G.zeros([3, 0, 4], np.float32))
    assert got.shape == (3, 0, 4)


def test_arange_linspace_identity(H, G):
    """Tensor.fs:3813-3886.  arange 1 1 10 has nine elements (BaseTests.fs:55); arange 1 2 10 has four (RatTests.fs:127)."""
    for dt in NUM:
        for args in ((1, 1, 10), (1, 2, 10), (0, 3, 100), (5, 1, 5)):
            ref, got = both(H, G, lambda x: type(x).arange(*args, x.Dev, x.DataType), np.zeros(1, dt))
            assert_exact(ref, got)
            assert_exact(np.arange(args[0], args[0] + len(got) * args[1], args[1]).astype(dt), got)
            assert len(got) == max(0, (args[2] - args[0]) // args[1])
        ref, got = both(H, G, lambda x: type(x).identity(37, x.Dev, x.DataType), np.zeros(1, dt))
        assert_exact(ref, got)
        assert_exact(np.eye(37, dtype=dt), got)
    for dt in (np.float32, np.float64):
        ref, got = both(H, G, lambda x: type(x).linspace(0, 5, 11, x.Dev, x.DataType), np.zeros(1, dt))
        assert_exact(ref, got)
        np.testing.assert_allclose(got, np.linspace(0, 5, 11), rtol=1e-6)
    with pytest.raises(ValueError):
        G.Dev and type(G.zeros([1], np.float32)).linspace(0, 1, 1, G.Dev, np.float32)


def test_empty_and_scalar(H, G):
    ref, got = both(H, G, lambda a, b: a + b, np.zeros((0, 5), np.float32), np.zeros((0, 5), np.float32))
    assert got.shape == (0, 5)
    ref, got = both(H, G, lambda a, b: a * b, np.array(3.0, np.float64), np.array(4.0, np.float64))
    assert got == 12.0 and ref == 12.0


def test_config1_chain_small(H, G, rng):
    """y = tanh(a*b + c); exp(-y*y) — the element-wise chain of the first benchmark configuration, six backend calls."""
    a, b, c = (rng.uniform(-1, 1, (256, 512)).astype(np.float32) for _ in range(3))

    def chain(a, b, c):
        y = (a * b + c).tanh()
        return (-(y * y)).exp()
    ref, got = both(H, G, chain, a, b, c)
    assert_rel(ref, got, 1e-6)
