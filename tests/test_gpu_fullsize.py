"""GPU: the five benchmark configurations at their FULL sizes, checked through facts that do not need the (slow) oracle:
IEEE-exact element ops and order-independent reductions against NumPy bit for bit, reordered sums against the fp64 sum within
the stated bound, compaction/gather/scatter against NumPy indexing, dot against the K-term bound, softmax rows summing to one."""
import numpy as np
import pytest

from util import assert_exact

pytestmark = pytest.mark.gpu


def test_config1_chain_4096(H, G):
    rng = np.random.default_rng(123)
    a, b, c = (rng.uniform(-1, 1, (4096, 4096)).astype(np.float32) for _ in range(3))

    def chain(a, b, c):
        t2 = a * b + c
        y = t2.tanh()
        return t2, (-(y * y)).exp()
    t2, out = (G.toNumpy(t) for t in chain(G.ofNumpy(a), G.ofNumpy(b), G.ofNumpy(c)))
    assert_exact(a * b + c, t2)                                   # separate multiply and add, no contraction
    ref_t2, ref_out = (H.toNumpy(t) for t in chain(H.ofNumpy(a), H.ofNumpy(b), H.ofNumpy(c)))
    assert_exact(ref_t2, t2)
    err = np.abs(out.astype(np.float64) - ref_out.astype(np.float64)) / np.abs(ref_out.astype(np.float64))
    assert err.max() <= 1e-6, err.max()


def test_config2_permuted_broadcast_add_and_copy(G):
    rng = np.random.default_rng(123)
    x = rng.standard_normal((256, 512, 1024), dtype=np.float32)
    v = rng.random(1024, dtype=np.float32)
    tx, tv = G.ofNumpy(x), G.ofNumpy(v)
    xp = tx.permuteAxes([2, 0, 1])                               # shape [512, 1024, 256], strides [1024, 1, 524288]
    assert xp.Shape == [512, 1024, 256] and xp.Stride == [1024, 1, 524288]
    y = G.toNumpy(xp + tv[None, :, None])
    want = np.transpose(x, (1, 2, 0)) + v[None, :, None]
    assert_exact(want, y)
    del y, want
    assert_exact(np.ascontiguousarray(np.transpose(x, (1, 2, 0))), G.toNumpy(xp.Copy()))
    # the NumPy reading of "axes (2,0,1)"
    xq = tx.permuteAxes([1, 2, 0])
    assert xq.Shape == [1024, 256, 512]
    assert_exact(np.transpose(x, (2, 0, 1)) + v[:, None, None], G.toNumpy(xq + tv[:, None, None]))


def test_large_transposing_tiles_operand_order_types_and_modes(G):
    """The large-tile transposing kernel (taken from 2048 tiles of 256 x 128 on) with the permuted operand first and second, a full
    second operand, a row-wise and an element-wise broadcast one, a bool result and a converting copy; NumPy is the checker."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((256, 256, 1024), dtype=np.float32)
    w = rng.standard_normal((256, 1024, 256), dtype=np.float32)
    tx, tw = G.ofNumpy(x), G.ofNumpy(w)
    xp = tx.permuteAxes([2, 0, 1])                               # shape [256, 1024, 256], strides [1024, 1, 262144]
    assert xp.Shape == [256, 1024, 256] and xp.Stride == [1024, 1, 262144]
    xt = np.transpose(x, (1, 2, 0))
    assert_exact(xt - w, G.toNumpy(xp - tw))
    assert_exact(w - xt, G.toNumpy(tw - xp))
    assert_exact(xt > w, G.toNumpy(xp > tw))
    r = rng.random(256, dtype=np.float32)
    assert_exact(r[None, None, :] - xt, G.toNumpy(G.ofNumpy(r)[None, None, :] - xp))
    v = rng.random(1024, dtype=np.float32)
    assert_exact(v[None, :, None] - xt, G.toNumpy(G.ofNumpy(v)[None, :, None] - xp))
    del w, tw
    i = rng.integers(-2 ** 24, 2 ** 24, (256, 256, 1024), dtype=np.int32)
    ip = G.ofNumpy(i).permuteAxes([2, 0, 1])
    assert_exact(np.ascontiguousarray(np.transpose(i, (1, 2, 0))).astype(np.float32), G.toNumpy(ip.convert(np.float32)))


def test_large_transposing_tiles_long_rows(G):
    """The 128 x 256 tiles that transposes with long target rows take from 2048 tiles on: a plain 2-D transpose, both operand
    orders, a row-wise operand and a bool result."""
    rng = np.random.default_rng(8)
    x = rng.standard_normal((8192, 8192), dtype=np.float32)
    w = rng.standard_normal((8192, 8192), dtype=np.float32)
    tx, tw = G.ofNumpy(x), G.ofNumpy(w)
    assert_exact(np.ascontiguousarray(x.T), G.toNumpy(tx.T.Copy()))
    assert_exact(x.T - w, G.toNumpy(tx.T - tw))
    assert_exact(w - x.T, G.toNumpy(tw - tx.T))
    assert_exact(x.T < w, G.toNumpy(tx.T < tw))
    v = rng.random(8192, dtype=np.float32)
    assert_exact(v[:, None] - x.T, G.toNumpy(G.ofNumpy(v)[:, None] - tx.T))
    assert_exact(x.T - v[None, :], G.toNumpy(tx.T - G.ofNumpy(v)[None, :]))


def test_large_transposing_tiles_double_precision(G):
    """The same kernel on 8-byte elements (two elements per 16-byte group, 128 x 128 tiles): short target rows with a row-wise
    operand, long rows with a second operand in either position, a bool result."""
    rng = np.random.default_rng(10)
    x = rng.standard_normal((256, 128, 1024))
    tx = G.ofNumpy(x)
    xp = tx.permuteAxes([2, 0, 1])                               # shape [128, 1024, 256]
    assert xp.Shape == [128, 1024, 256]
    xt = np.transpose(x, (1, 2, 0))
    assert_exact(np.ascontiguousarray(xt), G.toNumpy(xp.Copy()))
    v = rng.random(1024)
    assert_exact(xt - v[None, :, None], G.toNumpy(xp - G.ofNumpy(v)[None, :, None]))
    del x, tx, xp, xt
    y = rng.standard_normal((4096, 8192))
    z = rng.standard_normal((8192, 4096))
    ty, tz = G.ofNumpy(y), G.ofNumpy(z)
    assert_exact(np.ascontiguousarray(y.T), G.toNumpy(ty.T.Copy()))
    assert_exact(y.T - z, G.toNumpy(ty.T - tz))
    assert_exact(z - y.T, G.toNumpy(tz - ty.T))
    assert_exact(y.T >= z, G.toNumpy(ty.T >= tz))
    i = rng.integers(-2 ** 62, 2 ** 62, (4096, 8192), dtype=np.int64)
    assert_exact(np.ascontiguousarray(i.T), G.toNumpy(G.ofNumpy(i).T.Copy()))


def test_transposing_calls_on_ragged_shapes(G):
    """Transposing calls at full size on extents that are not multiples of the tiles: target rows that are not whole vectors
    (250 elements), a second operand of the target's shape, a row-wise one, a bool result; NumPy is the checker."""
    rng = np.random.default_rng(9)
    x = rng.standard_normal((250, 500, 1000), dtype=np.float32)
    tx = G.ofNumpy(x)
    xp = tx.permuteAxes([2, 0, 1])                               # shape [500, 1000, 250], strides [1000, 1, 500000]
    assert xp.Shape == [500, 1000, 250]
    xt = np.transpose(x, (1, 2, 0))
    assert_exact(np.ascontiguousarray(xt), G.toNumpy(xp.Copy()))
    v = rng.random(1000, dtype=np.float32)
    assert_exact(xt - v[None, :, None], G.toNumpy(xp - G.ofNumpy(v)[None, :, None]))
    w = rng.standard_normal((500, 1000, 250), dtype=np.float32)
    tw = G.ofNumpy(w)
    assert_exact(w - xt, G.toNumpy(tw - xp))
    assert_exact(xt <= w, G.toNumpy(xp <= tw))
    del w, tw, x, tx, xp, xt
    # 2-d, long rows: 9000 x 7000 -> 7000 x 9000 (edge tiles on both sides, whole vectors)
    y = rng.standard_normal((9000, 7000), dtype=np.float32)
    z = rng.standard_normal((7000, 9000), dtype=np.float32)
    ty, tz = G.ofNumpy(y), G.ofNumpy(z)
    assert_exact(np.ascontiguousarray(y.T), G.toNumpy(ty.T.Copy()))
    assert_exact(y.T - z, G.toNumpy(ty.T - tz))
    # ... and rows of 9001 elements in the target (element stores), the source's rows still whole vectors
    y2 = rng.standard_normal((9001, 7000), dtype=np.float32)
    assert_exact(np.ascontiguousarray(y2.T), G.toNumpy(G.ofNumpy(y2).T.Copy()))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_config3_reductions_8192(G, dt):
    rng = np.random.default_rng(123)
    x = rng.standard_normal((8192, 8192)).astype(dt) if dt == np.float32 else rng.uniform(-1, 1, (8192, 8192))
    t = G.ofNumpy(x)
    u = np.finfo(dt).eps / 2
    x64 = x.astype(np.float64)
    for ax in (1, 0):
        assert_exact(np.max(x, axis=ax), G.toNumpy(t.maxAxis(ax)))
        assert_exact(np.argmax(x, axis=ax).astype(np.int64), G.toNumpy(t.argMaxAxis(ax)))
        s = G.toNumpy(t.sumAxis(ax)).astype(np.float64)
        S = np.abs(x64).sum(axis=ax)
        assert np.all(np.abs(s - x64.sum(axis=ax)) <= (8192 + 64) * u * S)
    total = float(t.sum())
    assert abs(total - x64.sum()) <= (x.size + 64) * u * np.abs(x64).sum()
    # the tree is far tighter than the bound the sequential reference needs: within 64 u S
    assert abs(total - x64.sum()) <= 64 * u * np.abs(x64).sum()
    # a checksum of checksums: sum of row sums == sum of column sums == full sum (to the tree's accuracy)
    rows = G.toNumpy(t.sumAxis(1)).astype(np.float64).sum()
    cols = G.toNumpy(t.sumAxis(0)).astype(np.float64).sum()
    assert abs(rows - cols) <= 128 * u * np.abs(x64).sum()


def test_config4_indexing_16M(G):
    rng = np.random.default_rng(123)
    N, M = 1 << 24, 1 << 22
    a = rng.integers(-1000, 1001, N).astype(np.int32)
    b = rng.integers(-1000, 1001, N).astype(np.int32)
    idx = rng.integers(0, N, M).astype(np.int64)
    idxu = rng.permutation(N)[:M].astype(np.int64)
    ta, tb = G.ofNumpy(a), G.ofNumpy(b)
    T = type(ta)
    m = ta > 0
    assert_exact(a > 0, G.toNumpy(m))
    assert_exact(np.where(a > 0, a, b), G.toNumpy(T.ifThenElse(m, ta, tb)))
    assert m.countTrue() == int((a > 0).sum())
    assert_exact(a[a > 0], G.toNumpy(ta.M(m)))
    g = T.gather([G.ofNumpy(idx)], ta)
    assert_exact(a[idx], G.toNumpy(g))
    s = G.toNumpy(T.scatter([G.ofNumpy(idxu)], [N], g))
    want = np.zeros(N, np.int32)
    want[idxu] = a[idx]
    assert_exact(want, s)
    # masked set is the inverse of masked get
    z = G.zeros([N], np.int32)
    z.setM([m], ta.M(m))
    assert_exact(np.where(a > 0, a, 0).astype(np.int32), G.toNumpy(z))
    # trueIdx of the mask lists the selected positions in order
    assert_exact(np.flatnonzero(a > 0).astype(np.int64).reshape(-1, 1), G.toNumpy(m.trueIdx()))


def test_masked_get_many_blocks(G):
    """More than 8192 compaction blocks: exercises the scan launch instead of the in-kernel prefix."""
    rng = np.random.default_rng(7)
    n = 40_000_000
    a = rng.integers(-1000, 1001, n).astype(np.int32)
    ta = G.ofNumpy(a)
    assert_exact(a[a > 500], G.toNumpy(ta.M(ta > 500)))


def test_true_indices_many_blocks(G):
    """A dense 2-d mask of 144 Mi elements: more than 8192 blocks on the fast TrueIndices path (scan launch), sparse selection."""
    rng = np.random.default_rng(9)
    m = rng.random((9216, 16384)) < 0.01
    got = G.toNumpy(G.ofNumpy(m).trueIdx())
    assert_exact(np.argwhere(m).astype(np.int64), got)


def test_config5_mlp_block(G):
    rng = np.random.default_rng(123)
    sd = 1.0 / np.sqrt(512.0)
    a = (rng.standard_normal((64, 512, 512)) * sd).astype(np.float32)
    b = (rng.standard_normal((64, 512, 512)) * sd).astype(np.float32)
    ta, tb = G.ofNumpy(a), G.ofNumpy(b)
    c = ta @ tb
    cn = G.toNumpy(c)
    u = 2.0 ** -24
    for i in (0, 17, 63):                                        # fp64 truth on a few batches (the full fp64 product is slow on CPU)
        exact = a[i].astype(np.float64) @ b[i].astype(np.float64)
        S = np.abs(a[i]).astype(np.float64) @ np.abs(b[i]).astype(np.float64)
        assert np.all(np.abs(cn[i] - exact) <= 16 * u * S)      # measured 3.1 u S; a dropped partial product costs 10 u S and more
    t = c.tanh()
    mx = t.maxAxis(2)
    e = (t - mx[:, :, None]).exp()
    sm = e.sumAxis(2)
    p = G.toNumpy(e / sm[:, :, None])
    assert_exact(np.max(G.toNumpy(t), axis=2), G.toNumpy(mx))
    assert np.allclose(p.sum(axis=2, dtype=np.float64), 1.0, atol=1e-5)
    assert p.min() > 0 and p.max() < 1
    ref = np.exp(np.tanh(cn.astype(np.float64)) - np.tanh(cn.astype(np.float64)).max(axis=2, keepdims=True))
    ref /= ref.sum(axis=2, keepdims=True)
    assert np.allclose(p, ref, rtol=2e-5, atol=0)


def test_in_place_elementwise_at_64M_elements(G):
    """The target may be one of the sources (the reference's in-place forms, e.g. FillMultiply a a b,
    Tensor.Docs/articles/Guide-Operations.md:103-115): 8192 x 8192 single precision, target = first source, target = second
    source, and target = both, against NumPy bit for bit."""
    rng = np.random.default_rng(5)
    n = 8192
    a = rng.standard_normal((n, n), dtype=np.float32)
    b = rng.standard_normal((n, n), dtype=np.float32)
    ta, tb = G.ofNumpy(a), G.ofNumpy(b)
    ta.Backend.Multiply(ta, ta, tb)            # a <- a * b
    assert_exact(a * b, G.toNumpy(ta))
    tb.Backend.Subtract(tb, ta, tb)            # b <- (a * b) - b
    assert_exact(a * b - b, G.toNumpy(tb))
    ta.Backend.Add(ta, ta, ta)                 # a <- 2 (a * b)
    assert_exact((a * b) + (a * b), G.toNumpy(ta))
    ta.Backend.Tanh(ta, ta)
    ref = np.tanh(((a * b) + (a * b)).astype(np.float64)).astype(np.float32)
    got = G.toNumpy(ta)
    assert np.all(np.abs(got - ref) <= 1e-6 * np.abs(ref) + 1e-37)
    # a transposed view of the tensor itself as a source goes through a temporary on the host side of the interface as in the
    # reference; in place with the identical layout is the supported overlap
    tv = G.ofNumpy(a)
    tv.T.Backend.Abs(tv.T, tv.T)
    assert_exact(np.abs(a), G.toNumpy(tv))
