"""GPU parity: dot (vec.vec, mat.vec, mat.mat, batched) through the C ABI.
The reference's fp32/fp64 dot runs in MKL, whose summation order cannot be recovered, so the contract is the K-term
bound: with u = unit roundoff, S_ij = sum_k |a_ik||b_kj|, |gpu - oracle| <= (2K + 64) * u * S_ij and likewise against the fp64 product."""
import numpy as np
import pytest

from util import both

pytestmark = pytest.mark.gpu


def check_dot(ref, got, a, b):
    u = np.finfo(a.dtype).eps / 2
    K = a.shape[-1]
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    if b.ndim == 1:
        exact = a64 @ b64
        S = np.abs(a64) @ np.abs(b64)
    else:
        exact = np.matmul(a64, b64)
        S = np.matmul(np.abs(a64), np.abs(b64))
    bound = (2 * K + 64) * u * S + np.finfo(a.dtype).tiny
    assert got.shape == exact.shape
    assert np.all(np.abs(got.astype(np.float64) - ref.astype(np.float64)) <= bound)
    assert np.all(np.abs(got.astype(np.float64) - exact) <= bound)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("m,k,n", [(5, 3, 3), (128, 16, 128), (128, 512, 128), (256, 64, 384), (130, 70, 50), (1, 1, 1), (33, 1000, 7),
                                     # one, two, three and four K steps of 16 with a partial last one (the fetches run two steps ahead)
                                     (256, 20, 256), (64, 31, 300), (200, 33, 100), (300, 47, 260), (257, 49, 129)])
def test_matmat(H, G, rng, dt, m, k, n, tile_form):
    a = rng.standard_normal((m, k)).astype(dt)
    b = rng.standard_normal((k, n)).astype(dt)
    ref, got = both(H, G, lambda a, b: a @ b, a, b)
    check_dot(ref, got, a, b)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_empty_dimensions(H, G, dt):
    """An empty inner dimension gives zeros (an empty sum), empty outer dimensions give an empty result; nothing is fetched."""
    for m, k, n in [(5, 0, 7), (130, 0, 129), (0, 4, 3), (3, 4, 0)]:
        a = np.zeros((m, k), dt)
        b = np.zeros((k, n), dt)
        ref, got = both(H, G, lambda a, b: a @ b, a, b)
        assert got.shape == (m, n) and ref.shape == (m, n)
        assert np.array_equal(got, np.zeros((m, n), dt)) and np.array_equal(ref, got)
    a = np.zeros((2, 3, 0), dt)
    b = np.zeros((2, 0, 4), dt)
    ref, got = both(H, G, lambda a, b: a @ b, a, b)
    assert np.array_equal(got, np.zeros((2, 3, 4), dt)) and np.array_equal(ref, got)
    av = np.zeros((6, 0), dt)
    v = np.zeros((0,), dt)
    ref, got = both(H, G, lambda a, b: a @ b, av, v)
    assert np.array_equal(got, np.zeros((6,), dt)) and np.array_equal(ref, got)


def test_doc_vector(H, G):
    # Guide-Operations.md:129-148
    h = 3.0 * np.arange(5.0)[:, None] + np.arange(3.0)[None, :]
    i = 0.1 + np.eye(3)
    ref, got = both(H, G, lambda a, b: a @ b, h, i)
    exp = np.array([[0.3, 1.3, 2.3], [4.2, 5.2, 6.2], [8.1, 9.1, 10.1], [12.0, 13.0, 14.0], [15.9, 16.9, 17.9]])
    assert np.allclose(got, exp, rtol=1e-14)
    assert np.allclose(ref, exp, rtol=1e-14)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_vecvec_matvec(H, G, rng, dt):
    a = rng.standard_normal((77, 300)).astype(dt)
    x = rng.standard_normal(300).astype(dt)
    y = rng.standard_normal(300).astype(dt)
    ref, got = both(H, G, lambda a, x: a @ x, a, x)
    check_dot(ref, got, a, x)
    ref, got = both(H, G, lambda x, y: x @ y, x, y)
    check_dot(ref.reshape(1), got.reshape(1), x[None, :], y)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("shape_a,shape_b", [
    ((700, 900), (900, 650)),          # few tiles, long K: K is cut into chunks, the last one ragged
    ((128, 20000), (20000, 128)),      # one tile, many chunks (the wide finish)
    ((130, 4099), (4099, 70)),         # edge tiles in m and n, K not a multiple of the K step
    ((3, 2, 100, 1500), (3, 2, 1500, 60)),   # batch dimensions in front of the chunk dimension
])
def test_split_k(H, G, rng, dt, shape_a, shape_b, tile_form):
    """Products with few output tiles are cut along K and their partials added in chunk order: same bound as the uncut product,
    for contiguous operands, for transposed views (the strided kernel) and for a strided target."""
    a = rng.standard_normal(shape_a).astype(dt)
    b = rng.standard_normal(shape_b).astype(dt)
    ref, got = both(H, G, lambda a, b: a @ b, a, b)
    check_dot(ref, got, a, b)
    at = np.ascontiguousarray(np.swapaxes(a, -1, -2))
    bt = np.ascontiguousarray(np.swapaxes(b, -1, -2))
    ref, got = both(H, G, lambda a, b: a.T @ b.T, at, bt)
    check_dot(ref, got, a, b)

    def into_transposed_target(a, b):
        shp = list(a.Shape[:-2]) + [b.Shape[-1], a.Shape[-2]]
        t = type(a).new(shp, a.Dev, a.DataType)
        t.T.FillDot(a, b)
        return t
    ref, got = both(H, G, into_transposed_target, a, b)
    check_dot(np.swapaxes(ref, -1, -2), np.swapaxes(got, -1, -2), a, b)
    # the same call twice gives the same bits (fixed chunk order, no atomics)
    ta, tb = G.ofNumpy(a), G.ofNumpy(b)
    assert np.array_equal(G.toNumpy(ta @ tb), G.toNumpy(ta @ tb))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_batched_equals_loop_and_broadcast(H, G, rng, dt, tile_form):
    # Tensor.Test/BaseTests.fs:84-96: a batched product equals the loop of 2-d products
    a = rng.standard_normal((3, 4, 128, 48)).astype(dt)
    b = rng.standard_normal((3, 4, 48, 130)).astype(dt)
    ref, got = both(H, G, lambda a, b: a @ b, a, b)
    check_dot(ref, got, a, b)
    ta, tb = G.ofNumpy(a), G.ofNumpy(b)
    for i in range(3):
        for j in range(4):
            single = G.toNumpy(ta[i, j] @ tb[i, j])
            assert np.array_equal(single, got[i, j])
    # broadcast batch dimension (stride 0) and transposed operand views
    b1 = rng.standard_normal((1, 4, 48, 130)).astype(dt)
    ref, got = both(H, G, lambda a, b: a @ b, a, b1)
    check_dot(ref, got, a, np.broadcast_to(b1, (3, 4, 48, 130)))
    at = np.ascontiguousarray(np.swapaxes(a, -1, -2))
    ref, got = both(H, G, lambda a, b: a.T @ b, at, b)
    check_dot(ref, got, a, b)
    # (AB)^T = B^T A^T through transposed views on both sides and a transposed target
    def f(a, b):
        t = type(a).new([3, 4, 130, 128], a.Dev, a.DataType)
        t.FillDot(b.T, a.T)
        return t
    ref2, got2 = both(H, G, f, a, b)
    check_dot(np.swapaxes(ref2, -1, -2), np.swapaxes(got2, -1, -2), a, b)


def test_config5_block_small(H, G, rng, tile_form):
    """batched matmul -> tanh -> row softmax (max, subtract, exp, sum, divide), the fifth benchmark configuration."""
    a = (rng.standard_normal((4, 128, 128)) / np.sqrt(128)).astype(np.float32)
    b = (rng.standard_normal((4, 128, 128)) / np.sqrt(128)).astype(np.float32)

    def block(a, b):
        t = (a @ b).tanh()
        mx = t.maxAxis(2)
        e = (t - mx[:, :, None]).exp()
        sm = e.sumAxis(2)
        return e / sm[:, :, None]
    ref, got = both(H, G, block, a, b)
    assert np.allclose(got, ref, rtol=2e-4, atol=1e-7)
    assert np.allclose(got.sum(axis=2), 1.0, atol=1e-5)


def test_bool_dot_not_supported(G):
    a = G.ofNumpy(np.ones((4, 4), np.bool_))
    with pytest.raises(NotImplementedError):
        a @ a


@pytest.mark.parametrize("dt", [np.uint8, np.int8, np.int16, np.uint16, np.int32, np.uint32, np.int64, np.uint64])
def test_integer_dot_wraps_like_the_host_backend(H, G, rng, dt):
    """The reference's host backend computes dot of the types BLAS does not cover as multiply + sumAxis in the element type
    (Host/HostBackend.fs:544-546): wrapping arithmetic, so the result is bit-exact whatever the summation order."""
    info = np.iinfo(dt)

    def rnd(shape):
        return rng.integers(info.min, info.max, size=shape, dtype=dt, endpoint=True)
    for sa, sb in [((5, 3), (3, 3)), ((70, 130), (130, 65)), ((64, 300), (300, 64)), ((1, 1000), (1000, 1)), ((3, 2, 33, 40), (3, 2, 40, 17))]:
        a, b = rnd(sa), rnd(sb)
        ref, got = both(H, G, lambda a, b: a @ b, a, b)
        assert ref.dtype == got.dtype == dt and np.array_equal(ref, got)
        with np.errstate(over="ignore"):
            assert np.array_equal(got, np.matmul(a, b))          # numpy's integer matmul wraps the same way
    # transposed views, broadcast batch dimension, vector forms (strided vector), empty inner dimension
    a, b = rnd((40, 33)), rnd((40, 17))
    ref, got = both(H, G, lambda a, b: a.T @ b, a, b)
    assert np.array_equal(ref, got)
    a, b = rnd((4, 20, 30)), rnd((1, 30, 10))
    ref, got = both(H, G, lambda a, b: a @ b, a, b)
    assert np.array_equal(ref, got)
    m, v = rnd((300, 5000)), rnd((10000,))
    ref, got = both(H, G, lambda m, v: m @ v[0:10000][1:10000].reshape([9999])[0:5000], m, v)
    assert np.array_equal(ref, got)
    u, w = rnd((100000,)), rnd((100000,))
    ref, got = both(H, G, lambda u, w: u @ w, u, w)
    assert ref.shape == got.shape == () and np.array_equal(ref, got)
    ref, got = both(H, G, lambda a, b: a @ b, np.zeros((5, 0), dt), np.zeros((0, 7), dt))
    assert np.array_equal(got, np.zeros((5, 7), dt)) and np.array_equal(ref, got)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_vector_forms_layouts_and_sizes(H, G, rng, dt):
    """MatVecDot / VecVecDot on the dedicated reduction kernels: row-major and transposed matrices, strided and offset vectors,
    ragged and long K (split over several blocks)."""
    for m, k in [(1, 1), (3, 5), (257, 1030), (2000, 64), (5, 70001), (4096, 4099)]:
        a = rng.standard_normal((m, k)).astype(dt)
        x = rng.standard_normal(k).astype(dt)
        ref, got = both(H, G, lambda a, x: a @ x, a, x)
        check_dot(ref, got, a, x)
        # transposed view of a k-by-m matrix (m has stride 1)
        at = np.ascontiguousarray(a.T)
        ref, got = both(H, G, lambda at, x: at.T @ x, at, x)
        check_dot(ref, got, a, x)
    a = rng.standard_normal((300, 200)).astype(dt)
    x2 = rng.standard_normal((200, 3)).astype(dt)
    ref, got = both(H, G, lambda a, x: a[10:290, 5:195] @ x[5:195, 1], a, x2)        # offsets and a strided vector
    check_dot(ref, got, a[10:290, 5:195], x2[5:195, 1])
    u = rng.standard_normal(1_000_003).astype(dt)
    v = rng.standard_normal(1_000_003).astype(dt)
    ref, got = both(H, G, lambda u, v: u @ v, u, v)
    check_dot(ref.reshape(1), got.reshape(1), u[None, :], v)
    ref, got = both(H, G, lambda u, v: u[::1][3:100000] @ v.reverseAxis(0)[3:100000], u, v)
    check_dot(ref.reshape(1), got.reshape(1), u[None, 3:100000], v[::-1][3:100000])
    # a target with a stride (a column of a matrix)
    def f(a, x):
        t = type(a).new([300, 4], a.Dev, a.DataType)
        t.FillConst(0)
        t[:, 2].FillDot(a, x)
        return t
    ref, got = both(H, G, f, a, x2[:, 0].copy())
    check_dot(ref[:, 2], got[:, 2], a, x2[:, 0])
    assert (got[:, [0, 1, 3]] == 0).all()


@pytest.mark.parametrize("shape_a,shape_b", [((200, 64), (64, 300)), ((384, 16), (16, 256)), ((3, 130, 48), (3, 48, 257)),
                                             ((2, 2, 128, 32), (2, 2, 32, 128)), ((1500, 96), (96, 1100))])
def test_single_precision_on_bf16_parts(H, G, rng, shape_a, shape_b, tile_form):
    """Row-major single-precision products whose K is a multiple of 16 and that are not split along K run on the bf16 matrix
    instructions with every float cut into three bf16 parts.  Same contract as the fp32 instructions, and in practice the same
    accuracy: within 16 u S of the fp64 product for these sizes (the fp32 instructions measure 4-8 u S)."""
    for dist in ("normal", "positive"):
        a = (rng.standard_normal(shape_a) if dist == "normal" else rng.random(shape_a)).astype(np.float32)
        b = (rng.standard_normal(shape_b) if dist == "normal" else rng.random(shape_b)).astype(np.float32)
        ref, got = both(H, G, lambda a, b: a @ b, a, b)
        check_dot(ref, got, a, b)
        exact = np.matmul(a.astype(np.float64), b.astype(np.float64))
        S = np.matmul(np.abs(a).astype(np.float64), np.abs(b).astype(np.float64))
        assert np.all(np.abs(got - exact) <= 16 * 2.0 ** -24 * S)


def _views(G, a, b, ta, tb):
    """Device operands of a @ b, each uploaded as is or as its transpose and read back through a transposed view (the kernel's
    two stagings: k contiguous, or the other dimension contiguous)."""
    x = G.ofNumpy(np.ascontiguousarray(np.swapaxes(a, -1, -2))).T if ta else G.ofNumpy(a)
    y = G.ofNumpy(np.ascontiguousarray(np.swapaxes(b, -1, -2))).T if tb else G.ofNumpy(b)
    return x, y


def _err_over_uS(a, b, got):
    exact = np.matmul(a.astype(np.float64), b.astype(np.float64))
    S = np.matmul(np.abs(a).astype(np.float64), np.abs(b).astype(np.float64))
    return np.abs(got.astype(np.float64) - exact) / (2.0 ** -24 * S + 1e-300)


STAGINGS = [(False, False), (True, False), (False, True), (True, True)]


@pytest.mark.parametrize("m,k,n", [(256, 64, 256),      # whole tiles, one launch
                                   (700, 900, 650),     # cut along K into chunks
                                   (130, 4099, 70)])    # edge tiles, ragged K, chunks
def test_single_precision_special_values_follow_ieee(H, G, rng, m, k, n, tile_form):
    """Infinite, NaN, denormal-range and very small elements in the default single-precision product: the reference's sgemm forms
    IEEE products and sums (Host/HostBackend.fs:513-546), so inf x finite = +-inf, inf x 0 = NaN, inf - inf = NaN, NaN stays NaN.
    The class of every output (NaN / +inf / -inf / finite) must equal the oracle's and NumPy's, finite outputs keep the K-term bound."""
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    a[3, 5] = np.inf            # row 3: +-inf by the sign of b[5, :] ...
    b[5, 11] = 0.0              # ... except inf x 0 = NaN
    a[7, 2] = np.nan            # row 7: NaN
    b[4, 9] = -np.inf           # column 9: -+inf by the sign of a[:, 4]
    a[20, 4] = np.inf           # inf x -inf = -inf at (20, 9)
    a[100, k - 1] = -np.inf     # last k: row 100 ...
    b[k - 1, 33] = np.inf       # ... and column 33; (100, 33) = -inf
    a[101, 0], a[101, 1] = np.inf, -np.inf
    b[0, 40], b[1, 40] = 1.0, 1.0   # inf - inf = NaN at (101, 40)
    a[50, 7] = 1e-40            # a denormal and a very small normal element: finite results
    a[60, 8] = 2e-38
    want = H.toNumpy(H.ofNumpy(a) @ H.ofNumpy(b))
    with np.errstate(all="ignore"):
        want_np = a @ b
    assert np.isnan(want[3, 11]) and np.isnan(want[101, 40]) and np.all(np.isnan(want[7])) and want[20, 9] == -np.inf and want[100, 33] == -np.inf
    assert np.all(np.isinf(np.delete(want[3], [9, 11, 33])))
    for ta, tb in STAGINGS:
        x, y = _views(G, a, b, ta, tb)
        got = G.toNumpy(x @ y)
        for w in (want, want_np):
            assert np.array_equal(np.isnan(got), np.isnan(w)), (ta, tb)
            assert np.array_equal(np.isposinf(got), np.isposinf(w)) and np.array_equal(np.isneginf(got), np.isneginf(w)), (ta, tb)
        fin = np.isfinite(want)
        af, bf = np.where(np.isfinite(a), a, 0).astype(np.float64), np.where(np.isfinite(b), b, 0).astype(np.float64)
        S = np.abs(af) @ np.abs(bf)
        exact = af @ bf
        assert np.all(np.abs(got[fin] - exact[fin]) <= (2 * k + 64) * 2.0 ** -24 * S[fin])
        assert np.all(np.abs(got[fin] - want[fin]) <= (2 * k + 64) * 2.0 ** -24 * S[fin])
    # the largest finite values survive the cut into parts
    big = np.full((128, 16), 3e38, np.float32)
    pick = np.zeros((16, 128), np.float32)
    pick[0] = 1
    assert np.all(G.toNumpy(G.ofNumpy(big) @ G.ofNumpy(pick)) == np.float32(3e38))


@pytest.mark.parametrize("scale", [1e-30, 1e-33, 1e-36, 1e-38])
def test_single_precision_small_operands_keep_their_precision(G, rng, scale, tile_form):
    """Elements below 2^-109 cannot be cut into three bf16 parts exactly (the lowest part would fall below the smallest bf16
    denormal); tiles that hold such elements are computed on the fp32 instruction instead: same tight bound as O(1) data."""
    a = (rng.standard_normal((256, 512)) * scale).astype(np.float32)
    b = (rng.standard_normal((512, 384)) * 100).astype(np.float32)
    for ta, tb in STAGINGS[:3]:
        x, y = _views(G, a, b, ta, tb)
        assert _err_over_uS(a, b, G.toNumpy(x @ y)).max() <= 16
        x, y = _views(G, b.T.copy(), a.T.copy(), ta, tb)   # the small operand on the right
        assert _err_over_uS(b.T, a.T, G.toNumpy(x @ y)).max() <= 16


def test_single_precision_denormal_operands_and_sums(G, rng, tile_form):
    """Denormal operands (below 2^-126) are honoured; products and partial sums that are themselves below 2^-126 may be flushed
    to zero by the matrix instruction.  Stated bound: K x 2^-126 of absolute error on top of the K-term bound."""
    d = np.full((128, 16), 1e-40, np.float32)
    e = np.full((16, 128), 1e3, np.float32)
    assert np.array_equal(G.toNumpy(G.ofNumpy(d) @ G.ofNumpy(e)), d @ e)          # denormal x 1000: normal products, exact sums
    a = (rng.standard_normal((128, 64)) * 1e-41).astype(np.float32)
    b = (rng.standard_normal((64, 128)) * 100).astype(np.float32)
    for scale_some in (False, True):
        if scale_some:
            a[:, ::2] = (rng.standard_normal((128, 32)) * 1e-30).astype(np.float32)
        got = G.toNumpy(G.ofNumpy(a) @ G.ofNumpy(b)).astype(np.float64)
        a64, b64 = a.astype(np.float64), b.astype(np.float64)
        bound = (2 * 64 + 64) * 2.0 ** -24 * (np.abs(a64) @ np.abs(b64)) + 64 * 2.0 ** -126
        assert np.all(np.abs(got - a64 @ b64) <= bound)


@pytest.mark.parametrize("tiny", [2.0 ** -140, 2.0 ** -149, 2.0 ** -133, 1e-42, 2.0 ** -127])
def test_single_precision_smallest_denormal_operands(G, tiny, tile_form):
    """A denormal operand cannot be cut into bf16 parts (all its set bits lie in the low 16): its tile goes to the fp32 instruction,
    also when the element is so small that scaling it by 2^-17 rounds to zero.  tiny x 2^100 summed K times is a normal number that
    fp32 arithmetic gives exactly; every staging, both tile forms, one launch and chunks along K."""
    from deepnet_amd import native
    t32 = np.float32(tiny)
    assert t32 != 0
    for (m, k, n) in ((128, 16, 128), (256, 64, 384), (130, 4099, 70)):
        a = np.zeros((m, k), np.float32)
        b = np.full((k, n), 2.0 ** 100, np.float32)
        a[:, :16] = t32                       # sixteen equal terms: every partial sum is exact
        a[5, :] = 0
        a[5, 3] = t32                         # a single tiny element in an otherwise zero row
        want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
        assert np.all(want[0] == np.float32(16 * float(t32) * 2.0 ** 100)) and np.all(want[5] == np.float32(float(t32) * 2.0 ** 100))
        for ta, tb in STAGINGS:
            x, y = _views(G, a, b, ta, tb)
            assert np.array_equal(G.toNumpy(x @ y), want), (m, k, n, ta, tb)
            x, y = _views(G, np.ascontiguousarray(b.T), np.ascontiguousarray(a.T), ta, tb)   # the tiny operand on the right
            assert np.array_equal(G.toNumpy(x @ y), want.T), (m, k, n, ta, tb, "right")
        with native.option("dot_splits", 4):
            x, y = _views(G, a, b, False, False)
            assert np.array_equal(G.toNumpy(x @ y), want), (m, k, n, "chunks")


@pytest.mark.parametrize("k", [1, 2, 3, 4, 8, 15])
def test_single_precision_short_inner_dimension(H, G, rng, k):
    """K < 16 (outer products and the like) stays on the fp32 instruction: every product is one rounded fp32 product, so the
    result is within K roundings of the fp64 product (K = 1: the correctly rounded product itself, bit for bit)."""
    a = rng.standard_normal((200, k)).astype(np.float32)
    b = rng.standard_normal((k, 300)).astype(np.float32)
    for ta, tb in STAGINGS:
        x, y = _views(G, a, b, ta, tb)
        got = G.toNumpy(x @ y)
        assert _err_over_uS(a, b, got).max() <= k
        if k == 1:
            assert np.array_equal(got, a * b)


@pytest.mark.parametrize("shape_a,shape_b", [
    ((8, 512, 512), (8, 512, 512)),          # the benchmark's shape (a slice of its 64 pairs)
    ((1024, 4096), (4096, 1024)),            # long K, whole tiles
    ((1000, 4000), (4000, 1000)),            # long K, edge tiles
    ((700, 900), (900, 650)),                # split along K
    ((128, 20000), (20000, 128)),            # one tile, many chunks
    ((130, 4099), (4099, 70)),               # ragged K, chunks
    ((3, 2, 100, 1500), (3, 2, 1500, 60)),   # batch dimensions in front of the chunks
])
def test_single_precision_tight_bound_at_benchmark_shapes(G, rng, shape_a, shape_b, tile_form):
    """The bf16-parts kernel keeps six of the nine partial products.  A kernel that dropped one more (mid x mid, or a hi x lo) would
    be off by about 2^-16 |a||b| per product: 256 u, all of one sign for positive data, i.e. 50 u S and more at any K.  Measured:
    at most 3.2 u S for normal data and 11.2 u S for positive data (NumPy's sgemm on the same inputs: 3.0 and 14.5), so 16 u S is
    asserted for both, on both stagings."""
    for dist in ("normal", "positive"):
        a = (rng.standard_normal(shape_a) if dist == "normal" else rng.random(shape_a)).astype(np.float32)
        b = (rng.standard_normal(shape_b) if dist == "normal" else rng.random(shape_b)).astype(np.float32)
        for ta, tb in ((False, False), (True, True)):
            x, y = _views(G, a, b, ta, tb)
            worst = _err_over_uS(a, b, G.toNumpy(x @ y)).max()
            assert worst <= 16, (dist, ta, tb, worst)


@pytest.mark.parametrize("ta,tb", [(True, False), (False, True), (True, True)])
@pytest.mark.parametrize("m,k,n", [(200, 64, 300), (257, 100, 130), (1100, 40, 1500)])
def test_single_precision_on_bf16_parts_transposed_views(H, G, rng, ta, tb, m, k, n, tile_form):
    """Operands that are transposed views of row-major matrices take the same kernel with the other staging."""
    a = rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32)
    b = rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32)
    f = lambda x, y: (x.T if ta else x) @ (y.T if tb else y)
    ref, got = both(H, G, f, a, b)
    an, bn = (a.T if ta else a), (b.T if tb else b)
    check_dot(ref, got, an, bn)
    exact = an.astype(np.float64) @ bn.astype(np.float64)
    S = np.abs(an).astype(np.float64) @ np.abs(bn).astype(np.float64)
    assert np.all(np.abs(got - exact) <= 16 * 2.0 ** -24 * S)


def test_fp32_instruction_kernel_behind_the_switch(G):
    """dnh_set_option("dot_bf16x3", 0) sends single-precision products to the fp32 matrix instructions: same contract, same IEEE
    treatment of infinities; products of normal numbers are then single fp32 roundings, so K = 1 is exact."""
    from deepnet_amd import native
    rng = np.random.default_rng(3)
    assert native.get_option("dot_bf16x3") == 1
    with native.option("dot_bf16x3", 0):
        assert native.get_option("dot_bf16x3") == 0
        for (m, k, n) in ((200, 64, 300), (384, 16, 256), (130, 70, 50), (1024, 1024, 1024)):
            a = rng.standard_normal((m, k)).astype(np.float32)
            b = rng.standard_normal((k, n)).astype(np.float32)
            got = G.toNumpy(G.ofNumpy(a) @ G.ofNumpy(b)).astype(np.float64)
            exact = a.astype(np.float64) @ b.astype(np.float64)
            S = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
            assert np.all(np.abs(got - exact) <= (2 * k + 64) * 2.0 ** -24 * S), (m, k, n)
        a = np.ones((128, 16), np.float32)
        b = np.ones((16, 128), np.float32)
        a[3, 5] = np.inf
        got = G.toNumpy(G.ofNumpy(a) @ G.ofNumpy(b))
        assert np.all(np.isposinf(got[3])) and np.all(np.delete(got, 3, axis=0) == 16)
    assert native.get_option("dot_bf16x3") == 1
    with pytest.raises(ValueError):
        native.set_option("dot_bf16x3", 2)
    with pytest.raises(ValueError):
        native.set_option("no_such_switch", 1)


@pytest.mark.parametrize("ta,tb", STAGINGS)
@pytest.mark.parametrize("m,k,n", [(4096, 48, 4096),     # 256 tiles of 256 x 256: the large-tile kernel by the library's own choice
                                   (4000, 40, 4090),     # edge tiles on both sides and a partial last K step
                                   (4090, 24, 4000)])    # two K steps, the second partial: fetched before the loop starts
def test_single_precision_large_tiles(G, rng, ta, tb, m, k, n):
    """Products with at least a CU's worth of 256 x 256 tiles run the large-tile form of the bf16-parts kernel: same parts, same six
    products, so the same 16 u S; an infinite element sends its tile to the fp32 instructions, quarter by quarter."""
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    x, y = _views(G, a, b, ta, tb)
    assert _err_over_uS(a, b, G.toNumpy(x @ y)).max() <= 16
    a[300, 5] = np.inf           # tile row 1: quarter (1, *) of every tile in that row
    b[7, 1000] = -np.inf
    b[5, 2000] = 0.0             # inf x 0
    with np.errstate(all="ignore"):
        want = a @ b
    x, y = _views(G, a, b, ta, tb)
    got = G.toNumpy(x @ y)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isposinf(got), np.isposinf(want)) and np.array_equal(np.isneginf(got), np.isneginf(want))
    fin = np.isfinite(want)
    af, bf = np.where(np.isfinite(a), a, 0), np.where(np.isfinite(b), b, 0)
    assert _err_over_uS(af, bf, np.where(fin, got, 0))[fin].max() <= 16


@pytest.fixture(params=[-1, 1], ids=["tiles_auto", "tiles_256"])
def tile_form(request):
    """Runs a test once with the library's own choice of tile form and once with dot_big = 1, which sends every product that the
    bf16-parts kernel takes to its 256 x 256 form, whatever the size."""
    from deepnet_amd import native
    with native.option("dot_big", request.param):
        yield request.param


@pytest.mark.parametrize("ta,tb", STAGINGS)
@pytest.mark.parametrize("m,k,n", [(256, 8, 256), (257, 100, 130), (1100, 44, 1500), (300, 2049, 200)])
def test_double_precision_stagings(H, G, rng, ta, tb, m, k, n):
    """Double precision with row-major or transposed operands (the kernel's two stagings per operand), whole and partial K steps,
    edge tiles, one launch or chunks along K: IEEE products and sums in some order, so the K-term bound against the oracle and
    the exact product; an operand strided in both dimensions takes the general kernel and must agree as well."""
    a = rng.standard_normal((m, k))
    b = rng.standard_normal((k, n))
    x, y = _views(G, a, b, ta, tb)
    got = G.toNumpy(x @ y)
    ref = H.toNumpy(H.ofNumpy(a) @ H.ofNumpy(b))
    check_dot(ref, got, a, b)
    a[3, 5], b[5, 7] = np.inf, 0.0
    a[9, 1] = np.nan
    x, y = _views(G, a, b, ta, tb)
    got = G.toNumpy(x @ y)
    with np.errstate(all="ignore"):
        want = a @ b
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isposinf(got), np.isposinf(want))
    assert np.array_equal(np.isneginf(got), np.isneginf(want))
    # one plane of a 3-d tensor: strided in both dimensions
    wide = rng.standard_normal((m, k, 2))
    b2 = np.where(np.isfinite(b), b, 0.0)
    got = G.toNumpy(G.ofNumpy(wide)[:, :, 0] @ G.ofNumpy(b2))
    check_dot(wide[:, :, 0] @ b2, got, wide[:, :, 0], b2)


@pytest.mark.parametrize("dt", [np.int32, np.uint32, np.int64, np.uint64])
@pytest.mark.parametrize("ta,tb", STAGINGS)
@pytest.mark.parametrize("m,k,n", [(128, 32, 128), (130, 70, 50), (257, 1000, 300), (64, 4099, 33)])
def test_wide_integer_dot_on_the_int8_matrix_instruction(G, rng, dt, ta, tb, m, k, n):
    """32- and 64-bit integer products with K >= 32 are formed from signed byte planes on the int8 matrix instruction (the byte
    products that survive the modulus, one accumulator per shift): bit-identical to wrapping multiply + sum for every value,
    including the extremes, for both stagings of either operand, partial K steps and edge tiles; NumPy's integer matmul wraps
    the same way."""
    info = np.iinfo(dt)
    a = rng.integers(info.min, info.max, size=(m, k), dtype=dt, endpoint=True)
    b = rng.integers(info.min, info.max, size=(k, n), dtype=dt, endpoint=True)
    special = np.array([int(info.min), int(info.max), 0, 1, 127, 128, 255, 256, 0x7F7F7F7F, 0x80808080 & int(info.max), int(info.max) - 127,
                        0x7F7F7F7F7F7F7F7F & int(info.max), 0x8080808080808080 & int(info.max)], dtype=object).astype(dt)
    a[0, :special.size] = special
    a[1, :] = info.min
    b[:special.size, 0] = special[::-1]
    b[:, 1] = info.max
    if info.min < 0:
        a[2, :] = -1
        b[:, 2] = -1
        b[:, 3] = -128
    x, y = _views(G, a, b, ta, tb)
    got = G.toNumpy(x @ y)
    with np.errstate(over="ignore"):
        want = np.matmul(a, b)
    assert got.dtype == np.dtype(dt) and np.array_equal(got, want)


def test_64_bit_integer_dot_long_inner_dimension(G, rng):
    """More than 256 K steps: the int32 accumulators of the byte products are added into the 64-bit result before they can wrap.
    All-extreme operands make every byte product as large as it gets."""
    k = 20000
    for fill_a, fill_b in ((-2 ** 63, -2 ** 63), (2 ** 63 - 1, -2 ** 63), (-1, 2 ** 63 - 1), (0x7F7F7F7F7F7F7F7F, 0x7F7F7F7F7F7F7F7F)):
        a = np.full((40, k), fill_a, dtype=np.int64)
        b = np.full((k, 70), fill_b, dtype=np.int64)
        a[:, ::7] = rng.integers(-2 ** 63, 2 ** 63 - 1, size=a[:, ::7].shape, dtype=np.int64)
        with np.errstate(over="ignore"):
            want = np.matmul(a, b)
        assert np.array_equal(G.toNumpy(G.ofNumpy(a) @ G.ofNumpy(b)), want)
    u = rng.integers(0, 2 ** 64 - 1, size=(33, 9000), dtype=np.uint64)
    v = rng.integers(0, 2 ** 64 - 1, size=(9000, 65), dtype=np.uint64)
    with np.errstate(over="ignore"):
        assert np.array_equal(G.toNumpy(G.ofNumpy(u) @ G.ofNumpy(v)), np.matmul(u, v))


def test_32_bit_integer_dot_batched_and_large(G, rng):
    a = rng.integers(-2 ** 31, 2 ** 31 - 1, size=(3, 2, 200, 96), dtype=np.int32)
    b = rng.integers(-2 ** 31, 2 ** 31 - 1, size=(1, 2, 96, 150), dtype=np.int32)
    with np.errstate(over="ignore"):
        assert np.array_equal(G.toNumpy(G.ofNumpy(a) @ G.ofNumpy(b)), np.matmul(a, b))
    a = rng.integers(0, 2 ** 32 - 1, size=(1024, 2048), dtype=np.uint32)
    b = rng.integers(0, 2 ** 32 - 1, size=(2048, 1000), dtype=np.uint32)
    with np.errstate(over="ignore"):
        assert np.array_equal(G.toNumpy(G.ofNumpy(a) @ G.ofNumpy(b)), np.matmul(a, b))


import os as _os

_DOT_FUZZ = int(_os.environ.get("DNH_FUZZ_SEEDS_FACTOR", "1"))


@pytest.mark.parametrize("seed", range(24 * _DOT_FUZZ))
def test_dot_random_shapes_types_and_views(G, seed):
    """Random extents (tile edges, K tails, chunk counts and tile forms as the library chooses them), element types, transposed
    views and broadcast batch dimensions against NumPy: integers bit for bit (wrapping), floats within 16 u S of the fp64 product."""
    rng = np.random.default_rng(7000 + seed)
    for case in range(6):
        dt = [np.float32, np.float64, np.int32, np.int64, np.uint32, np.float32][int(rng.integers(0, 6))]
        big = rng.random() < 0.25
        m = int(rng.integers(1, 1500 if big else 300))
        n = int(rng.integers(1, 1500 if big else 300))
        k = int(rng.integers(1, 400 if big else 2500))
        batch = () if big or rng.random() < 0.5 else tuple(int(x) for x in rng.integers(1, 4, size=int(rng.integers(1, 3))))
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        bcast = len(batch) > 0 and rng.random() < 0.3
        sa = batch + (m, k)
        sb = ((1,) * len(batch) if bcast else batch) + (k, n)
        if np.dtype(dt).kind == "f":
            a = rng.standard_normal(sa).astype(dt)
            b = rng.standard_normal(sb).astype(dt)
        else:
            info = np.iinfo(dt)
            a = rng.integers(info.min, info.max, size=sa, dtype=dt, endpoint=True)
            b = rng.integers(info.min, info.max, size=sb, dtype=dt, endpoint=True)
        x, y = _views(G, a, b, ta, tb)
        got = G.toNumpy(x @ y)
        what = (seed, case, np.dtype(dt).name, sa, sb, ta, tb)
        if np.dtype(dt).kind == "f":
            u = np.finfo(dt).eps / 2
            exact = np.matmul(a.astype(np.float64), b.astype(np.float64))
            S = np.matmul(np.abs(a).astype(np.float64), np.abs(b).astype(np.float64))
            # fp64 results are compared with an fp64 product: leave room for its own rounding
            bound = (16 if dt == np.float32 else 2 * k + 64) * u * S + np.finfo(dt).tiny
            assert got.shape == exact.shape and np.all(np.abs(got - exact) <= bound), what
        else:
            with np.errstate(over="ignore"):
                want = np.matmul(a, b)
            assert got.dtype == np.dtype(dt) and np.array_equal(got, want), what


@pytest.mark.parametrize("dt", [np.float32, np.float64, np.int32, np.int64])
def test_dot_on_shifted_views_and_odd_pitches(G, dt):
    """Operands that are views starting at odd elements, with odd row pitches (k-contiguous rows fetched at element alignment),
    transposed and not, a K tail, a batch: integers bit for bit, floats within 16 u S (fp64: 2K + 64) of the fp64 product."""
    rng = np.random.default_rng(77)
    info = None if np.dtype(dt).kind == "f" else np.iinfo(dt)

    def rand(shape):
        if info is None:
            return rng.standard_normal(shape).astype(dt)
        return rng.integers(info.min, info.max, size=shape, dtype=dt, endpoint=True)

    def check(a, b, got, what):
        if info is None:
            u = np.finfo(dt).eps / 2
            exact = np.matmul(a.astype(np.float64), b.astype(np.float64))
            S = np.matmul(np.abs(a).astype(np.float64), np.abs(b).astype(np.float64))
            bound = (16 if dt == np.float32 else 2 * a.shape[-1] + 64) * u * S + np.finfo(dt).tiny
            assert got.shape == exact.shape and np.all(np.abs(got - exact) <= bound), what
        else:
            with np.errstate(over="ignore"):
                want = np.matmul(a, b)
            assert np.array_equal(got, want), what

    A = rand((517, 1003))
    B = rand((1003, 391))
    tA, tB = G.ofNumpy(A), G.ofNumpy(B)
    # a[1:, 3:] (513 x 1000, pitch 1003) . b[3:, 1:] (1000 x 390, pitch 391)
    check(A[1:, 3:], B[3:, 1:], G.toNumpy(tA[1:, 3:] @ tB[3:, 1:]), "row-major shifted")
    # a K tail: 997 inner elements
    check(A[2:, 5:1002], B[5:1002, 0:390], G.toNumpy(tA[2:, 5:1002] @ tB[5:1002, 0:390]), "K tail")
    # transposed shifted views: (B[3:, 1:]).T (390 x 1000, k strided) . (A[1:, 3:]).T (1000 x 516)
    check(B[3:, 1:].T, A[1:, 3:].T, G.toNumpy(tB[3:, 1:].T @ tA[1:, 3:].T), "transposed shifted")
    # matrix . vector and vector . vector on shifted views (rows and the transposed, column-wise form)
    x1 = rand((1003,))
    tx1 = G.ofNumpy(x1)
    check(A[1:, 3:], x1[3:], G.toNumpy(tA[1:, 3:] @ tx1[3:]), "matvec rows")
    check(A[1:, 3:].T, x1[1:518][:516], G.toNumpy(tA[1:, 3:].T @ tx1[1:517]), "matvec columns")
    check(x1[3:][None, :], x1[1:1001][:, None], np.asarray(G.toNumpy(tx1[3:] @ tx1[1:1001])).reshape(1, 1), "vecvec")
    # batched, odd pitches in every dimension
    C3 = rand((3, 131, 259))
    D3 = rand((3, 259, 67))
    got = G.toNumpy(G.ofNumpy(C3)[:, 1:, 2:] @ G.ofNumpy(D3)[:, 2:, 1:])
    check(C3[:, 1:, 2:], D3[:, 2:, 1:], got, "batched shifted")
