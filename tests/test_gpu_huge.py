"""GPU: tensors of more than 2^32 elements (uint8 / bool, 4.3 GB each).  Element positions no longer fit 32 bits, so every kernel
either computes 64-bit positions, is launched over pieces, or refuses with NotSupported; nothing may wrap around silently.  The data
has a prime period so that a position taken modulo 2^32 reads a different value."""
import numpy as np
import pytest

from util import assert_exact
from deepnet_amd.tensor import Tensor as T

pytestmark = pytest.mark.gpu

N = (1 << 32) + 4096


def pattern(n=N):
    block = np.random.default_rng(123).integers(0, 256, 1_000_003, dtype=np.uint8)
    return np.resize(block, n)


def test_elementwise_and_folds_beyond_32_bits(G):
    x = pattern()
    tx = G.ofNumpy(x)
    assert_exact(x + x, G.toNumpy(tx + tx))                         # flat kernel, wraps like uint8 on the host
    assert int(tx.sum()) == int(x.sum(dtype=np.uint8))              # one row longer than 2^32
    assert int(tx.max()) == 255
    m = tx > 127
    assert m.countTrue() == int(np.count_nonzero(x > 127))
    # rows of 2: 2^31 + 2048 outputs from the rows kernel, and the same through a transposed (strided) view
    r = tx.reshape([N // 2, 2])
    assert_exact(x.reshape(-1, 2).sum(axis=1, dtype=np.uint8), G.toNumpy(r.sumAxis(1)))
    assert_exact(x.reshape(-1, 2).max(axis=0), G.toNumpy(r.maxAxis(0)))
    # transposing copy with one extent beyond 2^31
    assert_exact(np.ascontiguousarray(x.reshape(-1, 2).T), G.toNumpy(r.T.Copy()))


def test_positions_beyond_32_bits(G):
    z = G.zeros([N], np.uint8)
    far = (1 << 32) + 100
    z[far] = 7
    assert z.argMax() == [far]
    assert int(G.toNumpy(z.findAxis(7, 0))) == far
    assert int(z[far].Value) == 7 and int(z[100].Value) == 0
    x = pattern()
    tx = G.ofNumpy(x)
    idx = np.array([far, 3, N - 1, 1 << 32], np.int64)
    assert_exact(x[idx], G.toNumpy(T.gather([G.ofNumpy(idx)], tx)))
    with pytest.raises(IndexError):
        T.gather([G.ofNumpy(np.array([N], np.int64))], tx)
    # scatter into a target of more than 2^32 int32 elements (17 GB), read back through gather and the full sum
    vals = np.array([5, -9, 1000, 11], np.int32)
    s = T.scatter([G.ofNumpy(idx)], [N], G.ofNumpy(vals))
    assert_exact(vals, G.toNumpy(T.gather([G.ofNumpy(idx)], s)))
    assert int(s.sum()) == int(vals.sum())
    del s
    # the same in single precision with a repeated index: the ordered form walks the 2^32 + 4096 cells in slabs of 4096 buckets
    fidx = np.array([far, 3, N - 1, 1 << 32, far, 3], np.int64)
    fvals = np.array([1e8, 0.5, -2.0, 7.25, 1.0, 1e-9], np.float32)
    fs = T.scatter([G.ofNumpy(fidx)], [N], G.ofNumpy(fvals))
    got = G.toNumpy(T.gather([G.ofNumpy(fidx[:4])], fs))
    want = np.array([np.float32(np.float32(0) + np.float32(1e8)) + np.float32(1.0), np.float32(0.5) + np.float32(1e-9), -2.0, 7.25], np.float32)
    assert_exact(want, got)


def test_compaction_beyond_32_bits_is_refused_not_wrapped(G):
    m = G.zeros([N], np.bool_)
    m[(1 << 32) + 5] = True
    x = G.zeros([N], np.uint8)
    with pytest.raises(NotImplementedError):
        x.M(m)
    with pytest.raises(NotImplementedError):
        m.trueIdx()
