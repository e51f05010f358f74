"""GPU parity for empty extents through every entry-point family: nothing to compute must mean nothing launched with a zero grid,
no division by an empty extent on the host, and the reference's results for empty folds (sum 0, product 1, max minValue,
min maxValue, all true, any false, countTrue 0, argMax / find NotFound: Tensor/Tensor/Host/ScalarOps.fs:606-665)."""
import numpy as np
import pytest

from util import both

pytestmark = pytest.mark.gpu

NOT_FOUND = -(2 ** 63) + 4   # SpecialIdx.NotFound, Tensor/Tensor/TensorRng.fs:24


def same(ref, got):
    assert ref.shape == got.shape and ref.dtype == got.dtype
    assert np.array_equal(ref, got)


@pytest.mark.parametrize("shape", [(0,), (3, 0), (0, 4), (2, 0, 5)])
@pytest.mark.parametrize("dt", [np.float32, np.int32, np.float64, np.uint8])
def test_elementwise_on_empty(H, G, dt, shape):
    a, b = np.zeros(shape, dt), np.ones(shape, dt)
    for f in (lambda a, b: a + b, lambda a, b: -a if a.DataType != np.uint8 else a * b, lambda a, b: a > b,
              lambda a, b: type(a).ifThenElse(a > b, a, b), lambda a, b: type(a).maxElemwise(a, b), lambda a, b: (a.T if a.NDims >= 2 else a).Copy(),
              lambda a, b: a.convert(np.int64)):
        ref, got = both(H, G, f, a, b)
        same(ref, got)
    # a scalar broadcast against an empty tensor stays empty
    ref, got = both(H, G, lambda a, b: a + b.flatten()[0:1].reshape([1] * a.NDims).broadcastTo(a.Shape) if b.NElems else a + a, a, b)
    same(ref, got)


@pytest.mark.parametrize("dt", [np.float32, np.float64, np.int32, np.int64, np.uint8])
def test_folds_over_an_empty_axis(H, G, dt):
    a = np.zeros((5, 0), dt)
    fp = np.issubdtype(dt, np.floating)
    lo = np.finfo(dt).min if fp else np.iinfo(dt).min
    hi = np.finfo(dt).max if fp else np.iinfo(dt).max
    cases = [(lambda x: x.sumAxis(1), 0), (lambda x: x.productAxis(1), 1), (lambda x: x.maxAxis(1), lo), (lambda x: x.minAxis(1), hi),
             (lambda x: x.argMaxAxis(1), NOT_FOUND), (lambda x: x.argMinAxis(1), NOT_FOUND), (lambda x: x.findAxis(0, 1), NOT_FOUND)]
    for f, want in cases:
        ref, got = both(H, G, f, a)
        same(ref, got)
        assert got.shape == (5,) and np.all(got == want)
    # the kept dimension is the empty one: empty results, no launch
    for f in (lambda x: x.sumAxis(0), lambda x: x.argMaxAxis(0), lambda x: x.maxAxis(0)):
        ref, got = both(H, G, f, a)
        same(ref, got)
        assert got.shape == (0,)
    # full folds of an empty tensor
    for f, want in ((lambda x: x.sumTensor(), 0), (lambda x: x.productTensor(), 1), (lambda x: x.maxTensor(), lo)):
        ref, got = both(H, G, f, a)
        same(ref, got)
        assert got.shape == () and got == want


def test_bool_folds_over_an_empty_axis(H, G):
    a = np.zeros((4, 0), np.bool_)
    for f, want in ((lambda x: x.allAxis(1), True), (lambda x: x.anyAxis(1), False), (lambda x: x.countTrueAxis(1), 0)):
        ref, got = both(H, G, f, a)
        same(ref, got)
        assert got.shape == (4,) and np.all(got == want)


@pytest.mark.parametrize("dt", [np.float32, np.int32, np.int64])
def test_gather_scatter_with_empty_index_tensors(H, G, dt):
    src = np.arange(12, dtype=dt).reshape(3, 4)
    i0 = np.zeros((0, 2), np.int64)
    i1 = np.zeros((0, 2), np.int64)
    ref, got = both(H, G, lambda s, a, b: type(s).gather([a, b], s), src, i0, i1)
    same(ref, got)
    assert got.shape == (0, 2)
    # scattering nothing leaves the zero-filled target
    vals = np.zeros((0, 2), dt)
    ref, got = both(H, G, lambda v, a, b: type(v).scatter([a, b], [3, 4], v), vals, i0, i1)
    same(ref, got)
    assert got.shape == (3, 4) and not got.any()
    # gathering from an empty source with empty indices
    ref, got = both(H, G, lambda s, a: type(s).gather([a], s), np.zeros((0,), dt), np.zeros((0,), np.int64))
    same(ref, got)


@pytest.mark.parametrize("dt", [np.float32, np.int64, np.uint8])
def test_masks_that_select_nothing(H, G, dt):
    a = np.arange(20, dtype=dt).reshape(4, 5)
    none2 = np.zeros((4, 5), np.bool_)
    ref, got = both(H, G, lambda x, m: x.M(m), a, none2)
    same(ref, got)
    assert got.shape == (0,)
    ref, got = both(H, G, lambda m: m.trueIdx(), none2)
    same(ref, got)
    assert got.shape == (0, 2)
    # per-dimension mask with no row selected, and masked assignment of nothing
    rows = np.zeros(4, np.bool_)
    ref, got = both(H, G, lambda x, r: x.M(r, None), a, rows)
    same(ref, got)
    assert got.shape == (0, 5)

    def set_nothing(x, m):
        y = x.Copy()
        y.setM([m], type(x).zeros([0], x.Dev, x.DataType))
        return y
    ref, got = both(H, G, set_nothing, a, none2)
    same(ref, got)
    assert np.array_equal(got, a)
    # empty source, empty mask
    ref, got = both(H, G, lambda x, m: x.M(m), np.zeros((0,), dt), np.zeros((0,), np.bool_))
    same(ref, got)


def test_creation_transfer_and_inversion_of_nothing(H, G):
    for M in (H, G):
        t = M.ofNumpy(np.zeros((0, 3), np.float32))
        assert M.toNumpy(type(t).zeros([0, 3], t.Dev, np.float32)).shape == (0, 3)
        assert M.toNumpy(M.ofNumpy(np.zeros((2, 0), np.int32))).shape == (2, 0)
        assert M.toNumpy(type(t).arange(5, 1, 5, t.Dev, np.int32)).shape == (0,)
        assert M.toNumpy(type(t).identity(0, t.Dev, np.float32)).shape == (0, 0)
    ref, got = both(H, G, lambda x: type(x).invert(x), np.zeros((3, 0, 0), np.float32))
    same(ref, got)
    ref, got = both(H, G, lambda x: type(x).invert(x), np.zeros((0, 2, 2), np.float64))
    same(ref, got)
