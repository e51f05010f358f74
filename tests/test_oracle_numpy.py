"""CPU: pins the oracle (oracle/hostref.cpp) against what the mathematics fixes, independently of its own formulas:
NumPy where NumPy is exactly specified (IEEE-exact element ops, first-occurrence argmax, sequential accumulate, fancy indexing),
closed forms and special values for transcendentals, brute force on tiny inputs, and structural identities for dot."""
import numpy as np
import pytest

from util import assert_exact, run_on

NOT_FOUND = -(2 ** 63) + 4
NUM = [np.uint8, np.int8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64, np.float32, np.float64]


def rnd(rng, dt, shape, lo=-50, hi=50):
    dt = np.dtype(dt)
    if dt.kind == "f":
        return (rng.random(shape) * (hi - lo) + lo).astype(dt)
    if dt.kind == "u":
        return rng.integers(0, 2 * hi, size=shape).astype(dt)
    return rng.integers(lo, hi, size=shape).astype(dt)


@pytest.mark.parametrize("dt", NUM)
def test_exact_binary_ops_match_numpy(H, rng, dt):
    a, b = rnd(rng, dt, (13, 37)), rnd(rng, dt, (13, 37))
    b[b == 0] = 3
    with np.errstate(all="ignore"):
        assert_exact((a + b).astype(dt), run_on(H, lambda x, y: x + y, [a, b]))
        assert_exact((a - b).astype(dt), run_on(H, lambda x, y: x - y, [a, b]))
        assert_exact((a * b).astype(dt), run_on(H, lambda x, y: x * y, [a, b]))
        assert_exact(np.maximum(a, b), run_on(H, lambda x, y: type(x).maxElemwise(x, y), [a, b]))
        assert_exact(np.minimum(a, b), run_on(H, lambda x, y: type(x).minElemwise(x, y), [a, b]))
        if np.dtype(dt).kind == "f":
            assert_exact(a / b, run_on(H, lambda x, y: x / y, [a, b]))
            assert_exact(np.fmod(a, b), run_on(H, lambda x, y: x % y, [a, b]))
        else:
            # .NET / and % truncate toward zero (C semantics), unlike NumPy's floor division
            q = np.trunc(a.astype(np.float64) / b.astype(np.float64)).astype(dt)
            assert_exact(q, run_on(H, lambda x, y: x / y, [a, b]))
            assert_exact((a.astype(np.int64) - q.astype(np.int64) * b.astype(np.int64)).astype(dt), run_on(H, lambda x, y: x % y, [a, b]))


def test_integer_overflow_wraps(H):
    a = np.array([2 ** 31 - 1, -2 ** 31, 2 ** 30], dtype=np.int32)
    b = np.array([1, -1, 4], dtype=np.int32)
    assert run_on(H, lambda x, y: x + y, [a, b]).tolist() == [-2 ** 31, 2 ** 31 - 1, 2 ** 30 + 4]
    assert run_on(H, lambda x, y: x * y, [a, b]).tolist() == [2 ** 31 - 1, -2 ** 31, 0]
    assert run_on(H, lambda x: x.sumAxis(0), [np.array([200, 100], np.uint8)]).tolist() == 44


def test_narrow_integer_division_follows_int32_arithmetic(H):
    """int16 (and int8) operands are divided as int32 and the quotient is truncated when stored (IL `div` then `conv.i2`): MinValue / -1
    wraps to MinValue, where the 32- and 64-bit types have no quotient (defined as 0, like a zero divisor)."""
    for dt, want in ((np.int16, -2 ** 15), (np.int8, -2 ** 7), (np.int32, 0), (np.int64, 0)):
        lo = np.iinfo(dt).min
        a, b = np.array([lo, lo, 5], dtype=dt), np.array([-1, 0, 0], dtype=dt)
        assert run_on(H, lambda x, y: x / y, [a, b]).tolist() == [want, 0, 0]
        assert run_on(H, lambda x, y: x % y, [a, b]).tolist() == [0, 0, 0]
    s = np.array([-300, 0, 17, -2 ** 15], dtype=np.int16)
    assert run_on(H, lambda x: x.sgn(), [s]).tolist() == [-1, 0, 1, -1]
    assert run_on(H, lambda x: abs(x), [s]).tolist() == [300, 0, 17, -2 ** 15]


def test_round_is_ties_to_even_and_sgn_abs(H):
    a = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 2.4999, -0.0], dtype=np.float64)
    assert run_on(H, lambda x: x.round(), [a]).tolist() == [0.0, 2.0, 2.0, -0.0, -2.0, -2.0, 2.0, -0.0]
    s = np.array([-3.5, -0.0, 0.0, 7.0, np.nan, -np.inf], dtype=np.float32)
    assert run_on(H, lambda x: x.sgn(), [s]).tolist() == [-1.0, 0.0, 0.0, 1.0, 0.0, -1.0]
    assert_exact(np.abs(s), run_on(H, lambda x: abs(x), [s]))
    assert_exact(np.ceil(a), run_on(H, lambda x: x.ceiling(), [a]))
    assert_exact(np.floor(a), run_on(H, lambda x: x.floor(), [a]))
    assert_exact(np.trunc(a), run_on(H, lambda x: x.truncate(), [a]))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_transcendental_closed_forms(H, dt):
    inf, nan = np.inf, np.nan
    x = np.array([0.0, inf, -inf, nan], dtype=dt)
    with np.errstate(all="ignore"):
        assert_exact(np.array([0.0, 1.0, -1.0, nan], dt), run_on(H, lambda t: t.tanh(), [x]))
        assert_exact(np.array([1.0, inf, 0.0, nan], dt), run_on(H, lambda t: t.exp(), [x]))
        assert_exact(np.array([0.0, dt(np.pi / 2), dt(-np.pi / 2), nan], dt), run_on(H, lambda t: t.atan(), [x]))
        assert_exact(np.array([-inf, inf, nan, nan], dt), run_on(H, lambda t: t.log(), [x]))
        assert_exact(np.array([0.0, inf, nan, nan], dt), run_on(H, lambda t: t.sqrt(), [x]))
    # fp32 functions are the double-precision libm result rounded to fp32 (F# Operators.<fn> on float32)
    rng = np.random.default_rng(5)
    v = rng.uniform(-3, 3, 2000).astype(dt)
    for name, npf in (("tanh", np.tanh), ("exp", np.exp), ("sin", np.sin), ("cos", np.cos), ("atan", np.arctan), ("sinh", np.sinh), ("cosh", np.cosh)):
        got = run_on(H, lambda t: getattr(t, name)(), [v])
        want = npf(v.astype(np.float64)).astype(dt)
        assert np.allclose(got, want, rtol=4 * np.finfo(dt).eps, atol=0), name
    # identities that a wrong formula breaks: exp(log x) = x, sin^2 + cos^2 = 1, tanh = sinh / cosh
    p = rng.uniform(0.1, 50, 500).astype(np.float64)
    assert np.allclose(run_on(H, lambda t: t.log().exp(), [p]), p, rtol=1e-14)
    assert np.allclose(run_on(H, lambda t: t.sin() * t.sin() + t.cos() * t.cos(), [p]), 1.0, rtol=1e-14)
    assert np.allclose(run_on(H, lambda t: t.sinh() / t.cosh(), [p / 10]), np.tanh(p / 10), rtol=1e-13)
    assert np.allclose(run_on(H, lambda t: t ** 2.0, [p]), p * p, rtol=1e-14)
    assert np.allclose(run_on(H, lambda t: t.log10(), [np.array([1e-3, 1.0, 1e5])]), [-3, 0, 5], atol=1e-15)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_sum_and_product_are_sequential_left_folds_in_T(H, rng, dt):
    """np.add.accumulate is a sequential fold in the array's dtype (np.sum is pairwise, and differs)."""
    x = rng.standard_normal((5, 4001)).astype(dt)
    want = np.add.accumulate(x, axis=1, dtype=dt)[:, -1]
    assert_exact(want, run_on(H, lambda t: t.sumAxis(1), [x]))
    want0 = np.add.accumulate(x, axis=0, dtype=dt)[-1, :]
    assert_exact(want0, run_on(H, lambda t: t.sumAxis(0), [x]))
    y = rng.uniform(0.9, 1.1, (3, 500)).astype(dt)
    assert_exact(np.multiply.accumulate(y, axis=1, dtype=dt)[:, -1], run_on(H, lambda t: t.productAxis(1), [y]))
    flat = np.add.accumulate(x.reshape(-1), dtype=dt)[-1]
    assert run_on(H, lambda t: t.sum(), [x]) == flat
    # thread count must not change any result (threads split dimension 0 only)
    H.set_threads(1)
    one = run_on(H, lambda t: t.sumAxis(1), [x])
    H.set_threads(0)
    assert_exact(want, one)


@pytest.mark.parametrize("dt", NUM)
def test_order_independent_folds_match_numpy(H, rng, dt):
    x = rnd(rng, dt, (7, 33, 5))
    for ax in range(3):
        assert_exact(np.max(x, axis=ax), run_on(H, lambda t: t.maxAxis(ax), [x]))
        assert_exact(np.min(x, axis=ax), run_on(H, lambda t: t.minAxis(ax), [x]))
        assert_exact(np.argmax(x, axis=ax).astype(np.int64), run_on(H, lambda t: t.argMaxAxis(ax), [x]))
        assert_exact(np.argmin(x, axis=ax).astype(np.int64), run_on(H, lambda t: t.argMinAxis(ax), [x]))
        if np.dtype(dt).kind != "f":
            assert_exact(np.add.reduce(x, axis=ax, dtype=dt), run_on(H, lambda t: t.sumAxis(ax), [x]))


def test_argmax_rule_brute_force(H):
    """State (NotFound, minValue); replace iff v > best: ties keep the lowest index, NaN never wins, rows that never exceed
    the initial value give NotFound (ScalarOps.fs:638-645)."""
    rows = [[1, 5, 5, 2, 5], [7, 7, 7, 7, 7], [-np.inf] * 5, [np.nan] * 5, [np.nan, 3, np.nan, 3, 1], [np.finfo(np.float32).min] * 5]
    x = np.array(rows, dtype=np.float32)

    def brute(row):
        best, pos = np.finfo(np.float32).min, NOT_FOUND
        for i, v in enumerate(row):
            if v > best:
                best, pos = v, i
        return pos
    with np.errstate(all="ignore"):
        assert run_on(H, lambda t: t.argMaxAxis(1), [x]).tolist() == [brute(r) for r in x]
    assert [brute(r) for r in x] == [1, 0, NOT_FOUND, NOT_FOUND, 1, NOT_FOUND]
    # max of a row of -inf is Single.MinValue, the fold's initial value (ScalarOps.fs:620-623)
    assert run_on(H, lambda t: t.maxAxis(1), [x[2:3]]).tolist() == [float(np.finfo(np.float32).min)]
    # empty axis: initial values
    e = np.zeros((2, 0), np.float32)
    assert run_on(H, lambda t: t.sumAxis(1), [e]).tolist() == [0.0, 0.0]
    assert run_on(H, lambda t: t.productAxis(1), [e]).tolist() == [1.0, 1.0]
    assert run_on(H, lambda t: t.argMaxAxis(1), [e]).tolist() == [NOT_FOUND, NOT_FOUND]


def test_bool_folds_and_find(H, rng):
    m = rng.random((9, 50)) < 0.5
    for ax in (0, 1):
        assert_exact(np.all(m, axis=ax), run_on(H, lambda t: t.allAxis(ax), [m]))
        assert_exact(np.any(m, axis=ax), run_on(H, lambda t: t.anyAxis(ax), [m]))
        assert_exact(np.count_nonzero(m, axis=ax).astype(np.int64), run_on(H, lambda t: t.countTrueAxis(ax), [m]))
    assert run_on(H, lambda t: t.all(), [np.zeros((0,), np.bool_)]) is True       # Guide-Logic.md:124-125
    assert run_on(H, lambda t: t.any(), [np.zeros((0,), np.bool_)]) is False
    x = rng.integers(0, 9, (20, 40)).astype(np.int32)
    want = np.array([next((i for i, v in enumerate(r) if v == 4), NOT_FOUND) for r in x], dtype=np.int64)
    assert_exact(want, run_on(H, lambda t: t.findAxis(4, 1), [x]))


def test_indexing_matches_numpy(H, rng):
    src = rng.integers(-100, 100, (30, 40)).astype(np.int32)
    i0 = rng.integers(0, 30, (5, 6)).astype(np.int64)
    i1 = rng.integers(0, 40, (5, 6)).astype(np.int64)
    assert_exact(src[i0, i1], run_on(H, lambda s, a, b: type(s).gather([a, b], s), [src, i0, i1]))
    j1 = rng.integers(0, 40, (30,)).astype(np.int64)
    assert_exact(src[np.arange(30), j1], run_on(H, lambda s, b: type(s).gather([None, b], s), [src, j1]))
    vals = rng.integers(0, 50, (5, 6)).astype(np.int32)
    want = np.zeros((30, 40), np.int32)
    np.add.at(want, (i0, i1), vals)
    assert_exact(want, run_on(H, lambda v, a, b: type(v).scatter([a, b], [30, 40], v), [vals, i0, i1]))
    m = rng.random((30, 40)) < 0.3
    assert_exact(src[m], run_on(H, lambda s, m: s.M(m), [src, m]))
    assert_exact(np.argwhere(m).astype(np.int64), run_on(H, lambda m: m.trueIdx(), [m]))
    m0, m1 = rng.random(30) < 0.5, rng.random(40) < 0.5
    assert_exact(src[np.ix_(m0, m1)], run_on(H, lambda s, a, b: s.M(a, b), [src, m0, m1]))
    with pytest.raises(IndexError):
        run_on(H, lambda s, a: type(s).gather([a, a], s), [src, np.array([40], dtype=np.int64)])


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_dot_against_fp64_and_identities(H, rng, dt):
    a = rng.standard_normal((2, 3, 17, 29)).astype(dt)
    b = rng.standard_normal((2, 3, 29, 11)).astype(dt)
    got = run_on(H, lambda x, y: x @ y, [a, b])
    exact = np.matmul(a.astype(np.float64), b.astype(np.float64))
    S = np.matmul(np.abs(a.astype(np.float64)), np.abs(b.astype(np.float64)))
    assert np.all(np.abs(got - exact) <= 29 * np.finfo(dt).eps * S)
    # batched product equals the loop of 2-d products (Tensor.Test/BaseTests.fs:84-96), bit for bit in this restatement
    for i in range(2):
        for j in range(3):
            assert_exact(run_on(H, lambda x, y: x @ y, [a[i, j], b[i, j]]), got[i, j])
    # (AB)^T = B^T A^T through transposed views; identity; matrix-vector and vector-vector forms
    ab_t = run_on(H, lambda x, y: y.T @ x.T, [a[0, 0], b[0, 0]])
    assert_exact(np.ascontiguousarray(got[0, 0].T), ab_t)
    eye = np.eye(29, dtype=dt)
    assert_exact(a[0, 0], run_on(H, lambda x, y: x @ y, [a[0, 0], eye]))
    mv = run_on(H, lambda x, y: x @ y, [a[0, 0], b[0, 0][:, 0].copy()])
    assert_exact(got[0, 0][:, 0].copy(), mv)
    vv = run_on(H, lambda x, y: x @ y, [a[0, 0][0].copy(), b[0, 0][:, 0].copy()])
    assert vv == got[0, 0][0, 0]


def test_convert_matches_numpy_casts(H, rng):
    for src in NUM:
        a = rnd(rng, src, (50,), 0, 100)
        for dst in NUM:
            assert_exact(a.astype(dst), run_on(H, lambda t: t.convert(dst), [a]))
        assert_exact(a != 0, run_on(H, lambda t: t.convert(np.bool_), [a]))
    assert run_on(H, lambda t: t.convert(np.int32), [np.array([2.9, -2.9, 0.5])]).tolist() == [2, -2, 0]


def test_errors_mirror_the_reference(H):
    a, b = H.ofNumpy(np.zeros((3, 4))), H.ofNumpy(np.zeros((5, 4)))
    with pytest.raises(ValueError):
        a + b                                   # shapes do not broadcast (TensorLayout.fs:246-254)
    with pytest.raises(ValueError):
        a @ b                                   # Tensor.fs:2796-2797
    with pytest.raises(NotImplementedError):
        H.ofNumpy(np.zeros(3, np.int32)).tanh()
    with pytest.raises(IndexError):
        a.sumAxis(2)


def test_convert_of_floats_outside_the_integer_range(H):
    """Pins the oracle's Convert rule for NaN, infinities and out-of-range floats against vectors worked out by hand
    (tests/convert_cases.py); in-range values truncate toward zero like a C cast."""
    import convert_cases as cc
    x = np.array(cc.INPUTS, dtype=np.float64)
    for dst in cc.EXPECTED:
        got = H.toNumpy(H.ofNumpy(x).convert(dst))
        assert got.dtype == np.dtype(dst)
        assert np.array_equal(got, cc.expected(dst)), (dst, got, cc.expected(dst))
    r = np.random.default_rng(2).uniform(-100, 100, 1000)
    for dst in (np.int32, np.int64, np.int8, np.int16):
        assert np.array_equal(H.toNumpy(H.ofNumpy(r).convert(dst)), np.trunc(r).astype(dst))


def test_max_min_folds_with_nans_follow_the_sequential_rule(H):
    """`if res > v then res else v` from minValue (Host/ScalarOps.fs:620-628), spelled out element by element: a NaN replaces the
    running value and is replaced by the next element, so the result is the fold of what follows the last NaN."""
    nan, inf = np.nan, np.inf
    x = np.array([[1, 5, 2, 4], [nan, 5, 2, 4], [1, nan, 2, 4], [1, 5, 2, nan], [nan, nan, nan, nan], [9, nan, -inf, -inf],
                  [nan, 3, nan, 3], [-inf, -inf, -inf, -inf]], dtype=np.float32)
    fmin, fmax = np.finfo(np.float32).min, np.finfo(np.float32).max
    want_max = np.array([5, 5, 4, nan, nan, -inf, 3, fmin], dtype=np.float32)
    want_min = np.array([1, 2, 2, nan, nan, -inf, 3, -inf], dtype=np.float32)
    got_max = run_on(H, lambda t: t.maxAxis(1), [x])
    got_min = run_on(H, lambda t: t.minAxis(1), [x])
    assert np.array_equal(got_max, want_max, equal_nan=True), got_max
    assert np.array_equal(got_min, want_min, equal_nan=True), got_min
    assert fmax > 0 and run_on(H, lambda t: t.minAxis(1), [np.array([[inf, inf]], np.float64)]).tolist() == [np.finfo(np.float64).max]
