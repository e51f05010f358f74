"""GPU parity: axis reductions through the C ABI against the CPU oracle.
Order-independent folds (max/min/all/any/countTrue, integer sums/products) and ArgMin/ArgMax/Find are bit-exact.
Float sums/products are re-associated on the GPU; contract (u = unit roundoff of T, S = sum of |x| over the reduced
elements, n their count):  |gpu - ref| <= (n + c + d) * u * S  with c + d <= 64 (per-lane chunk + tree depth bound)."""
import numpy as np
import pytest

from util import both, assert_exact

pytestmark = pytest.mark.gpu

NOT_FOUND = -(2 ** 63) + 4


def sum_bound_ok(ref, got, x, axis):
    u = np.finfo(x.dtype).eps / 2
    S = np.sum(np.abs(x.astype(np.float64)), axis=axis)
    n = x.shape[axis] if axis is not None else x.size
    bound = (n + 64) * u * S + np.finfo(x.dtype).tiny
    exact = np.sum(x.astype(np.float64), axis=axis)
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    assert np.all(err <= bound), f"worst {np.max(err / np.maximum(bound, 1e-300))} of bound"
    # the tree is expected to be at least as close to the exact sum as the sequential fold's own bound
    assert np.all(np.abs(got.astype(np.float64) - exact) <= bound)


SHAPES = [(7, 5), (64, 1000), (3, 4099), (1000, 33), (5, 17, 300), (2, 40000), (1, 70000)]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("shape", SHAPES)
def test_sum_max_min_fp_all_axes(H, G, rng, dt, shape):
    x = rng.standard_normal(shape).astype(dt)
    for ax in range(len(shape)):
        ref, got = both(H, G, lambda t: t.sumAxis(ax), x)
        sum_bound_ok(ref, got, x, ax)
        for name in ("maxAxis", "minAxis", "argMaxAxis", "argMinAxis"):
            ref, got = both(H, G, lambda t: getattr(t, name)(ax), x)
            assert_exact(ref, got)
        assert_exact(np.argmax(x, axis=ax).astype(np.int64), G.toNumpy(G.ofNumpy(x).argMaxAxis(ax)))
        assert_exact(np.max(x, axis=ax), G.toNumpy(G.ofNumpy(x).maxAxis(ax)))


@pytest.mark.parametrize("dt", [np.int32, np.int64, np.uint8, np.int8, np.int16, np.uint16, np.uint32, np.uint64])
def test_int_folds_exact(H, G, rng, dt):
    x = rng.integers(0, 100, size=(33, 1030)).astype(dt)
    for ax in (0, 1):
        for name in ("sumAxis", "productAxis", "maxAxis", "minAxis", "argMaxAxis", "argMinAxis"):
            ref, got = both(H, G, lambda t: getattr(t, name)(ax), x)
            assert_exact(ref, got)


def test_product_fp(H, G, rng):
    x = rng.uniform(0.9, 1.1, (50, 700)).astype(np.float32)
    for ax in (0, 1):
        ref, got = both(H, G, lambda t: t.productAxis(ax), x)
        assert np.allclose(ref, got, rtol=x.shape[ax] * 2 ** -23, atol=0)


def test_full_reductions(H, G, rng):
    x = rng.standard_normal((300, 1111)).astype(np.float32)
    ref, got = both(H, G, lambda t: t.sumTensor(), x)
    sum_bound_ok(ref, got, x, None)
    for f in (lambda t: t.maxTensor(), lambda t: t.minTensor()):
        ref, got = both(H, G, f, x)
        assert_exact(ref, got)
    t = G.ofNumpy(x)
    assert t.argMax() == list(np.unravel_index(np.argmax(x), x.shape))
    assert t.argMin() == list(np.unravel_index(np.argmin(x), x.shape))
    # a permuted view flattens through a copy (ITensor.fs:306-316)
    ref, got = both(H, G, lambda t: t.T.maxTensor(), x)
    assert_exact(ref, got)


def test_argmax_ties_and_notfound(H, G):
    x = np.array([[1, 5, 5, 2, 5], [7, 7, 7, 7, 7], [-np.inf] * 5, [np.nan] * 5, [np.nan, 3, np.nan, 3, 1]], dtype=np.float32)
    ref, got = both(H, G, lambda t: t.argMaxAxis(1), x)
    assert_exact(ref, got)
    assert got.tolist() == [1, 0, NOT_FOUND, NOT_FOUND, 1]
    ref, got = both(H, G, lambda t: t.argMinAxis(1), x)
    assert_exact(ref, got)
    # planted ties far apart in a long row: the lowest index must win whatever lane/block sees it
    y = np.zeros((4, 100000), dtype=np.float32)
    y[0, [99999, 512, 70000]] = 9
    y[1, [65536, 65537]] = 3
    y[2, 99999] = 1
    for ax_view in (lambda t: t.argMaxAxis(1), lambda t: t.T.Copy().argMaxAxis(0)):
        ref, got = both(H, G, ax_view, y)
        assert_exact(ref, got)
        assert got.tolist() == [512, 65536, 99999, 0]
    # integer rows that never exceed the initial value
    z = np.full((2, 10), np.iinfo(np.int32).min, dtype=np.int32)
    z[1, 7] = 0
    ref, got = both(H, G, lambda t: t.argMaxAxis(1), z)
    assert got.tolist() == [NOT_FOUND, 7]
    assert_exact(ref, got)


def test_max_of_neg_inf_is_min_value(H, G):
    # the fold starts at Single.MinValue, so a row of -inf yields -FLT_MAX (ScalarOps.fs:620-623)
    x = np.full((3, 100), -np.inf, dtype=np.float32)
    ref, got = both(H, G, lambda t: t.maxAxis(1), x)
    assert_exact(ref, got)
    assert got[0] == np.finfo(np.float32).min


def test_empty_axis_yields_initial_value(H, G):
    x = np.zeros((4, 0), dtype=np.float32)
    for name, val in (("sumAxis", 0.0), ("productAxis", 1.0), ("maxAxis", np.finfo(np.float32).min), ("minAxis", np.finfo(np.float32).max)):
        ref, got = both(H, G, lambda t: getattr(t, name)(1), x)
        assert_exact(ref, got)
        assert got.tolist() == [val] * 4
    ref, got = both(H, G, lambda t: t.argMaxAxis(1), x)
    assert got.tolist() == [NOT_FOUND] * 4
    b = np.zeros((3, 0), dtype=np.bool_)
    assert G.toNumpy(G.ofNumpy(b).allAxis(1)).tolist() == [True] * 3
    assert G.toNumpy(G.ofNumpy(b).anyAxis(1)).tolist() == [False] * 3
    assert G.toNumpy(G.ofNumpy(b).countTrueAxis(1)).tolist() == [0] * 3


@pytest.mark.parametrize("shape", [(9, 1000), (100, 100), (2, 3, 4097), (1, 300000)])
def test_bool_folds(H, G, rng, shape):
    m = rng.random(shape) < 0.5
    m2 = np.ones(shape, dtype=np.bool_)
    m2.flat[m2.size // 2] = False
    for x in (m, m2, np.zeros(shape, np.bool_)):
        for ax in range(len(shape)):
            for name in ("allAxis", "anyAxis", "countTrueAxis"):
                ref, got = both(H, G, lambda t: getattr(t, name)(ax), x)
                assert_exact(ref, got)
        assert G.ofNumpy(x).countTrue() == int(np.count_nonzero(x))
        assert G.ofNumpy(x).all() == bool(x.all()) and G.ofNumpy(x).any() == bool(x.any())


def test_find(H, G, rng):
    x = rng.integers(0, 50, size=(40, 5000)).astype(np.int32)
    for ax in (0, 1):
        ref, got = both(H, G, lambda t: t.findAxis(7, ax), x)
        assert_exact(ref, got)
    ref, got = both(H, G, lambda t: t.findAxis(1000, 1), x)
    assert (got == NOT_FOUND).all()
    assert_exact(ref, got)
    a = np.array([[1.0, 2.0, 3.0, 4.0], [5.0, 6.0, 7.0, 3.0]])
    assert G.toNumpy(G.ofNumpy(a).findAxis(3.0, 1)).tolist() == [2, 3]          # Guide-Index.md:52-57
    assert G.ofNumpy(a).tryFind(3.0) == [0, 2]                                   # Guide-Index.md:44-49


def test_strided_reduce_axis(H, G, rng):
    x = rng.standard_normal((50, 60, 70)).astype(np.float32)
    # reduce over a middle axis of a sliced, permuted view
    def f(t):
        v = t[5:45, :, 3:60].permuteAxes([1, 2, 0])
        return v.maxAxis(0), v.maxAxis(1), v.maxAxis(2), v.argMaxAxis(1)
    ref, got = both(H, G, f, x)
    for r, g in zip(ref, got):
        assert_exact(r, g)
    # a single strided column reduced to a scalar
    ref, got = both(H, G, lambda t: t[:, 7, 9].maxAxis(0), x)
    assert_exact(ref, got)


def _seq_fold(x, is_max):
    """The reference's sequential Max / Min fold (Host/ScalarOps.fs:620-628) over the last axis, element by element."""
    dt = x.dtype
    init = np.finfo(dt).min if is_max else np.finfo(dt).max
    out = np.empty(x.shape[:-1], dt)
    for idx in np.ndindex(*x.shape[:-1]):
        r = dt.type(init)
        for v in x[idx]:
            r = r if (r > v if is_max else r < v) else v
        out[idx] = r
    return out


@pytest.mark.parametrize("dt", [np.float32, np.float64, np.int32, np.int64])
def test_folds_of_shifted_views(G, rng, dt):
    """Folds over views that start at odd elements and have odd row pitches (their rows are fetched in vectors at element
    alignment): along both axes, row lengths with and without a vector tail; NumPy is the checker."""
    x = (rng.standard_normal((1025, 4099)) * 100).astype(dt)
    tx = G.ofNumpy(x)
    for (r0, r1, c0, c1) in [(0, 1025, 3, 4099), (1, 1025, 1, 4098), (2, 1001, 5, 2054)]:
        v, tv = x[r0:r1, c0:c1], tx[r0:r1, c0:c1]
        for ax in (1, 0):
            assert_exact(v.max(axis=ax), G.toNumpy(tv.maxAxis(ax)))
            assert_exact(v.argmax(axis=ax).astype(np.int64), G.toNumpy(tv.argMaxAxis(ax)))
            got = G.toNumpy(tv.sumAxis(ax))
            if np.dtype(dt).kind == "f":
                want = v.astype(np.float64).sum(axis=ax)
                bound = (v.shape[ax] + 64) * (np.finfo(dt).eps / 2) * np.abs(v.astype(np.float64)).sum(axis=ax)
                assert np.all(np.abs(got.astype(np.float64) - want) <= bound)
            else:
                assert_exact(v.sum(axis=ax, dtype=dt), got)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(37, 300), (3, 70000), (600, 40), (1, 5), (2000, 16), (40, 2, 513)])
def test_max_min_follow_the_sequential_rule_with_nans(H, G, rng, dt, shape):
    """With NaNs among the elements the reference's `if res > v then res else v` gives the fold of what follows the last NaN (NaN if
    it comes last).  Rows without a NaN, with one in front, in the middle, at the end, several, all NaN, NaN followed only by -inf;
    along the last axis and (through a transposed view) along the first; row, split-row and column forms of the kernels.  Bit for bit
    against the oracle, and against the rule spelled out in Python on the smaller shapes."""
    x = rng.standard_normal(shape).astype(dt)
    flat = x.reshape(-1, shape[-1])
    n = shape[-1]
    for i in range(flat.shape[0]):
        kind = i % 8
        if kind == 1: flat[i, 0] = np.nan
        elif kind == 2: flat[i, n // 2] = np.nan
        elif kind == 3: flat[i, n - 1] = np.nan
        elif kind == 4: flat[i, rng.integers(0, n, size=min(n, 5))] = np.nan
        elif kind == 5: flat[i, :] = np.nan
        elif kind == 6:
            flat[i, : n // 2 + 1] = np.nan
            flat[i, n // 2 + 1:] = -np.inf if i % 16 == 6 else np.inf
        elif kind == 7: flat[i, rng.integers(0, n)] = np.nan
    for name in ("maxAxis", "minAxis"):
        for axis_last in (True, False):
            def f(t):
                v = t if axis_last else t.permuteAxes(list(range(1, len(shape))) + [0])   # the reduced axis first, as a view
                return getattr(v, name)(len(shape) - 1 if axis_last else 0)
            ref, got = both(H, G, f, x)
            assert ref.dtype == got.dtype == np.dtype(dt)
            assert np.array_equal(ref, got, equal_nan=True), (name, axis_last)
            if x.size <= 40000 and axis_last:
                want = _seq_fold(x, name == "maxAxis")
                assert np.array_equal(want, got, equal_nan=True), name
    # the whole tensor as one row (the split-row form for the long shapes)
    ref, got = both(H, G, lambda t: t.max(), x)
    assert np.array_equal(ref, got, equal_nan=True)
    ref, got = both(H, G, lambda t: t.min(), x)
    assert np.array_equal(ref, got, equal_nan=True)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_max_min_with_nans_on_long_axes(H, G, dt):
    """NaNs in folds whose axis is cut into chunks (a whole tensor of 2^24 elements, a few rows of 2^20, a tall matrix reduced down
    its columns): the threads that share the row redo only the last chunk that holds a NaN.  NaN in the first chunk, in the middle,
    as the last element of a chunk that is followed by -inf only, as the very last element; bit for bit against the oracle."""
    import time
    rng = np.random.default_rng(5)
    n = 1 << 24
    base = rng.standard_normal(n).astype(dt)
    cases = {
        "front": [0], "middle": [n // 2 + 17], "last": [n - 1], "several": [5, n // 3, n - 70000],
        "chunk_end_then_neg_inf": [n // 2 - 1],
    }
    for name, where in cases.items():
        x = base.copy()
        x[where] = np.nan
        if name == "chunk_end_then_neg_inf":
            x[n // 2:] = -np.inf      # what follows the NaN is -inf only: Max is -inf (not minValue), Min is -inf
        for fold in ("max", "min"):
            ref, got = both(H, G, lambda t: getattr(t, fold)(), x)
            assert np.array_equal(ref, got, equal_nan=True), (name, fold, ref, got)
        rows = x.reshape(16, n // 16)
        cols = np.ascontiguousarray(x.reshape(n // 64, 64))
        for fold in ("maxAxis", "minAxis"):
            ref, got = both(H, G, lambda t: getattr(t, fold)(1), rows)
            assert np.array_equal(ref, got, equal_nan=True), (name, fold, "rows")
            ref, got = both(H, G, lambda t: getattr(t, fold)(0), cols)
            assert np.array_equal(ref, got, equal_nan=True), (name, fold, "columns")
    # one NaN in 2^26 elements must not turn the fold into a walk by a single thread (seconds): generous bound
    big = G.ofNumpy(np.concatenate([base] * 4))
    big[12345:12346].FillConst(float("nan"))
    big.max()
    t0 = time.perf_counter()
    got = big.max()
    assert time.perf_counter() - t0 < 0.25
    assert got == np.concatenate([base] * 4)[12346:].max()
