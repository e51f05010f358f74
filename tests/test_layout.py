"""CPU: the TensorLayout algebra (deepnet_amd/layout.py) against closed forms and NumPy's own view machinery."""
import numpy as np
import pytest

from deepnet_amd import layout as L
from deepnet_amd.layout import Rng, TensorLayout


def as_view(arr, lay):
    isz = arr.dtype.itemsize
    flat = arr.reshape(-1)
    return np.lib.stride_tricks.as_strided(flat[lay.Offset:], shape=lay.Shape, strides=[s * isz for s in lay.Stride])


def test_strides_and_contiguity():
    assert L.cStride([2, 3, 4]) == (12, 4, 1)
    assert L.fStride([2, 3, 4]) == (1, 2, 6)
    assert L.orderedStride([2, 3, 4], [1, 0, 2]) == (3, 1, 6)
    c = L.newC([2, 3, 4])
    assert L.isC(c) and not L.isF(c) and L.hasContiguousMemory(c)
    assert L.isF(L.newF([2, 3, 4]))
    assert L.isC(TensorLayout((1, 5), 0, (77, 1)))      # strides of extent-1 dimensions do not matter (TensorLayout.fs:127-130)
    with pytest.raises(ValueError):
        L.orderedStride([2, 3], [0, 0])


def test_permute_axes_moves_axis_i_to_position_perm_i():
    base = np.arange(4 * 2 * 3).reshape(4, 2, 3)
    lay = L.permuteAxes([2, 0, 1], L.newC(base.shape))
    assert lay.Shape == (2, 3, 4)                                            # Guide-Shape.md:82-83 has [4;2;2] -> [2;2;4]
    assert np.array_equal(as_view(base, lay), np.moveaxis(base, [0, 1, 2], [2, 0, 1]))
    # the second benchmark configuration's view
    x = L.permuteAxes([2, 0, 1], L.newC([256, 512, 1024]))
    assert x.Shape == (512, 1024, 256) and x.Stride == (1024, 1, 524288)
    with pytest.raises(ValueError):
        L.permuteAxes([0, 1], L.newC([2, 3, 4]))


def test_broadcast_pad_insert():
    a = L.newC([4, 3, 1])
    b = L.newC([2])
    pa, pb = L.broadcastToSame(a, b)
    assert pa.Shape == pb.Shape == (4, 3, 2)
    assert pa.Stride == (3, 1, 0) and pb.Stride == (0, 0, 1)
    assert L.isBroadcasted(pa) and not L.isBroadcasted(a)
    v = L.view([Rng.NewAxis, Rng.All, Rng.NewAxis], L.newC([1024]))
    assert v.Shape == (1, 1024, 1) and v.Stride == (0, 1, 0)
    assert L.broadcastToShape([512, 1024, 256], v).Stride == (0, 1, 0)
    assert L.insertAxis(1, L.newC([3, 4])).Shape == (3, 1, 4)
    assert L.padLeft(L.newC([3])).Shape == (1, 3) and L.padRight(L.newC([3])).Shape == (3, 1)
    assert L.cutLeft(L.newC([3, 4])).Shape == (4,) and L.cutRight(L.newC([3, 4])).Shape == (3,)
    with pytest.raises(ValueError):
        L.broadcastToSame(L.newC([3, 4]), L.newC([5, 4]))
    with pytest.raises(ValueError):
        L.broadcastToShape([3], L.newC([2, 3]))
    sas = L.broadcastToSameMany([L.newC([1, 5]), L.newC([4, 1]), L.newC([5])])
    assert [s.Shape for s in sas] == [(4, 5)] * 3


def test_views_match_numpy_slicing():
    base = np.arange(5 * 6 * 7).reshape(5, 6, 7)
    lay = L.newC(base.shape)
    v = L.view([Rng.Range(1, 3), Rng.Elem(2), Rng.Range(None, 4)], lay)      # F# ranges are inclusive
    assert np.array_equal(as_view(base, v), base[1:4, 2, :5])
    v2 = L.view([Rng.AllFill, Rng.Elem(3)], lay)
    assert np.array_equal(as_view(base, v2), base[..., 3])
    v3 = L.view([Rng.Elem(4), Rng.AllFill], lay)
    assert np.array_equal(as_view(base, v3), base[4])
    assert L.view([Rng.Range(3, 2), Rng.All, Rng.All], lay).Shape == (0, 6, 7)   # empty slice
    r = L.reverseAxis(1, lay)
    assert np.array_equal(as_view(base, r), base[:, ::-1, :])
    assert r.Stride[1] == -7 and r.Offset == 35
    d = L.diagAxis(0, 1, L.newC([4, 4]))
    assert np.array_equal(as_view(np.arange(16), d), np.diag(np.arange(16).reshape(4, 4)))
    with pytest.raises(IndexError):
        L.view([Rng.Elem(5), Rng.All, Rng.All], lay)
    with pytest.raises(IndexError):
        L.view([Rng.All], lay)


def test_reshape_rules():
    a = L.newC([2, 3, 4])
    assert L.reshape([6, 4], a).Stride == (4, 1)
    assert L.reshape([2, L.Remainder, 1], a).Shape == (2, 12, 1)
    t = L.transpose(L.newC([3, 4]))
    assert L.tryReshape([12], t) is None                     # needs a copy
    assert L.tryReshape([1, 4, 1, 3], t).Stride == (0, 1, 0, 4)   # singleton insertion keeps the view
    assert L.tryReshape([4, 3], L.transpose(L.newC([3, 4]))).Stride == (1, 4)
    with pytest.raises(ValueError):
        L.reshape([5, 5], a)
    with pytest.raises(ValueError):
        L.reshape([L.Remainder, L.Remainder], a)
    with pytest.raises(ValueError):
        L.reshape([7, L.Remainder], a)


def test_addr_and_linear_index():
    lay = TensorLayout((3, 4), 5, (1, 3))
    assert L.addr([2, 3], lay) == 5 + 2 + 9
    with pytest.raises(IndexError):
        L.addr([3, 0], lay)
    assert L.linearToIdx(L.newC([2, 3, 4]), 17) == [1, 1, 1]
    assert L.idxToLinear(L.newC([2, 3, 4]), [1, 1, 1]) == 17
    assert L.swapDim(0, 2, L.newC([2, 3, 4])).Shape == (4, 3, 2)


def test_frontend_views_round_trip_through_the_oracle_device(H):
    """Host <-> tensor round trips for C-order and non-C-order layouts (the reference's Tensor.Test/CudaTests.fs:28-51 idea)."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal((4, 5, 6))
    t = H.ofNumpy(x)
    assert np.array_equal(H.toNumpy(t.permuteAxes([2, 0, 1])), np.moveaxis(x, [0, 1, 2], [2, 0, 1]))
    assert np.array_equal(H.toNumpy(t[1:3, :, 2]), x[1:3, :, 2])
    assert np.array_equal(H.toNumpy(t.T.Copy()), np.swapaxes(x, 1, 2))
    assert np.array_equal(H.toNumpy(t.T.flatten()), np.swapaxes(x, 1, 2).reshape(-1))
    assert np.array_equal(H.toNumpy(t[None, 0, :, :]), x[None, 0, :, :])
    assert t[1, 2, 3].Value == x[1, 2, 3]
    col = t.Copy("ColumnMajor")
    assert col.Stride == [1, 4, 20] and np.array_equal(H.toNumpy(col), x)
