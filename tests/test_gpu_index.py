"""GPU parity: gather / scatter / masked get / masked set / trueIdx through the C ABI — all bit-exact against the oracle
and against NumPy's own indexing."""
import numpy as np
import pytest

from util import both, assert_exact

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [np.int32, np.float32, np.int64, np.float64, np.uint8, np.bool_, np.int16])
def test_gather_1d(H, G, rng, dt):
    src = (rng.integers(0, 2, 100000) > 0) if dt == np.bool_ else rng.integers(-1000, 1000, 100000).astype(dt)
    idx = rng.integers(0, src.size, 30011).astype(np.int64)
    ref, got = both(H, G, lambda s, i: type(s).gather([i], s), src, idx)
    assert_exact(ref, got)
    assert_exact(src[idx], got)


def test_gather_nd_with_none_and_broadcast(H, G, rng):
    src = rng.standard_normal((30, 40, 50)).astype(np.float32)
    i0 = rng.integers(0, 30, (40, 1)).astype(np.int64)
    i2 = rng.integers(0, 50, (1, 7)).astype(np.int64)
    # target shape [40, 7]; dimension 1 of src maps identically from target dimension 1?  No: identity needs d < target rank
    ref, got = both(H, G, lambda s, a, b: type(s).gather([a, None, b], s), src, i0, rng.integers(0, 50, (40, 40)).astype(np.int64))
    assert_exact(ref, got)
    # documentation vectors (Guide-Index.md:87-105)
    s = np.array([[0.0, 0.1, 0.2, 0.3], [1.0, 1.1, 1.2, 1.3], [2.0, 2.1, 2.2, 2.3]])
    g = G.toNumpy(type(G.ofNumpy(s)).gather([G.ofNumpy(np.array([1, 2, 0, 0])), G.ofNumpy(np.array([3, 1, 0, 3]))], G.ofNumpy(s)))
    assert g.tolist() == [1.3, 2.1, 0.0, 0.3]
    g2 = G.toNumpy(type(G.ofNumpy(s)).gather([None, G.ofNumpy(np.array([3, 1, 0]))], G.ofNumpy(s)))
    assert g2.tolist() == [0.3, 1.1, 2.0]
    _ = i2


def test_gather_out_of_range_raises(H, G):
    s = np.arange(10, dtype=np.int32)
    for bad in ([3, 10], [-1, 2]):
        with pytest.raises(IndexError):
            type(G.ofNumpy(s)).gather([G.ofNumpy(np.array(bad, dtype=np.int64))], G.ofNumpy(s))
        with pytest.raises(IndexError):
            type(H.ofNumpy(s)).gather([H.ofNumpy(np.array(bad, dtype=np.int64))], H.ofNumpy(s))
    # the flag is cleared by the read: a following valid gather succeeds
    ok = type(G.ofNumpy(s)).gather([G.ofNumpy(np.array([9, 0], dtype=np.int64))], G.ofNumpy(s))
    assert G.toNumpy(ok).tolist() == [9, 0]


@pytest.mark.parametrize("dt", [np.int32, np.int64, np.uint32, np.uint64, np.uint8, np.int8, np.int16, np.uint16])
def test_scatter_int_with_duplicates(H, G, rng, dt):
    src = rng.integers(0, 100, 50000).astype(dt)
    idx = rng.integers(0, 777, 50000).astype(np.int64)          # heavy duplication: sums, wrapping for narrow types
    ref, got = both(H, G, lambda s, i: type(s).scatter([i], [1000], s), src, idx)
    assert_exact(ref, got)
    exp = np.zeros(1000, dtype=dt)
    np.add.at(exp, idx, src)
    assert_exact(exp, got)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_scatter_fp_unique(H, G, rng, dt):
    src = rng.standard_normal(40000).astype(dt)
    idx = rng.permutation(100000)[:40000].astype(np.int64)
    ref, got = both(H, G, lambda s, i: type(s).scatter([i], [100000], s), src, idx)
    assert_exact(ref, got)


def _wide(rng, m, dt):
    """Values spread over twelve decades, both signs: the order of a cell's additions shows in the last bits of its sum."""
    return (rng.standard_normal(m) * 10.0 ** rng.uniform(-6, 6, m)).astype(dt)


def _check_fp_scatter_bound(got, idx, src, n, dt):
    """Stated bound of floating-point scatter (either form): a cell that m_j sources name is within m_j u sum|src_s| of the exact sum."""
    exact = np.zeros(n, np.float64)
    np.add.at(exact, idx, src.astype(np.float64))
    mag = np.zeros(n, np.float64)
    np.add.at(mag, idx, np.abs(src.astype(np.float64)))
    cnt = np.bincount(idx, minlength=n).astype(np.float64)
    u = np.finfo(dt).eps / 2
    assert np.all(np.abs(got.astype(np.float64) - exact) <= cnt * u * mag)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("m,n,kind", [
    (50_000, 777, "dup"),                      # about 64 sources per cell
    (70_000, 1, "dup"),                        # one cell takes everything: one run per batch
    (200_000, 5, "dup"),
    ((1 << 20) + 123, 300_000, "dup"),         # many workgroups feed every bucket
    (3 << 20, 5_000_000, "skewed"),            # most sources land in a few buckets, many buckets stay empty
    (8191, 100_000, "dup"), (8193, 9000, "dup"), (1, 10, "dup"),
    (1 << 20, 40_000_000, "dup"),              # a table of more than 4096 buckets: two slabs
])
def test_scatter_fp_with_duplicates_adds_in_source_order(H, G, rng, dt, m, n, kind):
    """Floating-point scatter with repeated indices: every cell receives its sources in row-major source order, as the reference's
    loop adds them, so the sums agree bit for bit with the oracle and with NumPy's unbuffered np.add.at (which is specified to apply
    the updates one after the other), and two runs give the same bits."""
    if kind == "skewed":
        idx = np.where(rng.random(m) < 0.9, rng.integers(0, 40_000, m), rng.integers(0, n, m)).astype(np.int64)
    else:
        idx = rng.integers(0, n, m).astype(np.int64)
    src = _wide(rng, m, dt)
    ref, got = both(H, G, lambda s, i: type(s).scatter([i], [n], s), src, idx)
    assert_exact(ref, got)
    exp = np.zeros(n, dtype=dt)
    np.add.at(exp, idx, src)
    assert_exact(exp, got)
    again = G.toNumpy(type(G.ofNumpy(src)).scatter([G.ofNumpy(idx)], [n], G.ofNumpy(src)))
    assert_exact(got, again)
    _check_fp_scatter_bound(got, idx, src, n, dt)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_scatter_fp_layouts_existing_values_and_bad_indices(H, G, rng, dt):
    """The ordered form on everything the entry point accepts: index tensors per dimension, a strided (transposed) source, a target
    that is a strided view holding values already, identity dimensions, out-of-range indices (reported, skipped, the rest lands)."""
    src = _wide(rng, 300 * 200, dt).reshape(300, 200)
    i0 = rng.integers(0, 50, (300, 200)).astype(np.int64)
    i1 = rng.integers(0, 60, (300, 200)).astype(np.int64)
    ref, got = both(H, G, lambda s, a, b: type(s).scatter([a, b], [50, 60], s), src, i0, i1)
    assert_exact(ref, got)
    exp = np.zeros((50, 60), dt)
    np.add.at(exp, (i0, i1), src)
    assert_exact(exp, got)
    # transposed source and index views (row-major order of the VIEW is the order of the additions)
    ref, got = both(H, G, lambda s, a, b: type(s).scatter([a.T, b.T], [50, 60], s.T), src, i0, i1)
    assert_exact(ref, got)
    exp = np.zeros((50, 60), dt)
    np.add.at(exp, (i0.T, i1.T), src.T)
    assert_exact(exp, got)
    # identity on dimension 0 (None), an index tensor for dimension 1
    j1 = rng.integers(0, 7, (300, 200)).astype(np.int64)
    ref, got = both(H, G, lambda s, b: type(s).scatter([None, b], [300, 7], s), src, j1)
    assert_exact(ref, got)
    # a strided target view with values in it
    before = _wide(rng, 3 * 1000, dt).reshape(1000, 3)
    idx = rng.integers(0, 1000, 20000).astype(np.int64)
    vals = _wide(rng, 20000, dt)
    exp = before.copy()
    np.add.at(exp[:, 1], idx, vals)
    for mod in (H, G):
        t = mod.ofNumpy(before)
        view = t[:, 1]                                         # one column: stride 3
        view.Backend.Scatter(view, [mod.ofNumpy(idx)], mod.ofNumpy(vals))
        assert_exact(exp, mod.toNumpy(t))
    # indices outside the table
    bad = idx.copy()
    bad[[5, 7000, 19999]] = [1000, -1, 2 ** 40]
    t2 = G.zeros([1000], dt)
    with pytest.raises(IndexError):
        t2.Backend.Scatter(t2, [G.ofNumpy(bad)], G.ofNumpy(vals))
    keep = np.ones(20000, bool)
    keep[[5, 7000, 19999]] = False
    exp2 = np.zeros(1000, dt)
    np.add.at(exp2, idx[keep], vals[keep])
    assert_exact(exp2, G.toNumpy(t2))


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_scatter_fp_atomic_form_behind_the_switch(G, rng, dt):
    """dnh_set_option("scatter_fp_atomic", 1) selects float atomics: the order of a cell's additions then varies from run to run, the
    stated bound still holds."""
    from deepnet_amd import native
    m, n = 300_000, 5000
    idx = rng.integers(0, n, m).astype(np.int64)
    src = _wide(rng, m, dt)
    with native.option("scatter_fp_atomic", 1):
        got = G.toNumpy(type(G.ofNumpy(src)).scatter([G.ofNumpy(idx)], [n], G.ofNumpy(src)))
    _check_fp_scatter_bound(got, idx, src, n, dt)


@pytest.mark.parametrize("dt", [np.int32, np.uint32])
@pytest.mark.parametrize("m,n,kind", [
    ((1 << 20) + 123, 300_000, "dup"),         # many updates per element; table not a whole number of buckets
    ((1 << 21), (1 << 22) + 5, "unique"),      # the benchmark's form at a quarter of its size, ragged table
    ((1 << 20) + 1, 16384, "dup"),             # one bucket
    ((1 << 20) + 7, 1, "dup"),                 # one element
    (3 << 20, 5_000_000, "skewed"),            # most updates land in a few buckets, many buckets stay empty
])
def test_scatter_many_updates_binned(H, G, rng, dt, m, n, kind):
    """Large scatters of 32-bit integers are sorted by bucket of the table and summed per bucket (a different kernel sequence
    from the direct one): bit-exact against the oracle's sequential loop and against np.add.at, sums wrapping."""
    if kind == "unique":
        idx = rng.permutation(n)[:m].astype(np.int64)
    elif kind == "skewed":
        idx = np.where(rng.random(m) < 0.9, rng.integers(0, 40_000, m), rng.integers(0, n, m)).astype(np.int64)
    else:
        idx = rng.integers(0, n, m).astype(np.int64)
    src = rng.integers(0, 2 ** 31 - 1, m).astype(dt)            # large values: sums wrap
    ref, got = both(H, G, lambda s, i: type(s).scatter([i], [n], s), src, idx)
    assert_exact(ref, got)
    exp = np.zeros(n, dtype=dt)
    np.add.at(exp, idx, src)
    assert_exact(exp, got)


def test_scatter_many_updates_adds_to_the_target_and_reports_bad_indices(G, rng):
    m, n = (1 << 20) + 5, 200_001
    idx = rng.integers(0, n, m).astype(np.int64)
    src = rng.integers(-1000, 1000, m).astype(np.int32)
    before = rng.integers(-5, 5, n + 3).astype(np.int32)
    t = G.ofNumpy(before)
    view = t[3:]                                                  # a target that is not 16-byte aligned, holding values already
    view.Backend.Scatter(view, [G.ofNumpy(idx)], G.ofNumpy(src))
    exp = before.copy()
    np.add.at(exp[3:], idx, src)
    assert_exact(exp, G.toNumpy(t))
    # indices outside the table: reported, skipped, everything else still lands
    bad = idx.copy()
    bad[[5, 70_000, m - 1]] = [n, -1, 2 ** 40]
    t2 = G.zeros([n], np.int32)
    with pytest.raises(IndexError):
        t2.Backend.Scatter(t2, [G.ofNumpy(bad)], G.ofNumpy(src))
    keep = np.ones(m, bool)
    keep[[5, 70_000, m - 1]] = False
    exp2 = np.zeros(n, np.int32)
    np.add.at(exp2, idx[keep], src[keep])
    assert_exact(exp2, G.toNumpy(t2))


def test_scatter_doc_vector(H, G):
    # Guide-Index.md:118-133: first row summed into [0,3]; rows 1 and 2 swapped; row 3 stays zero
    src = np.array([[0.0, 0.1, 0.2, 0.3], [1.0, 1.1, 1.2, 1.3], [2.0, 2.1, 2.2, 2.3]])
    i0 = np.array([[0, 0, 0, 0], [2, 2, 2, 2], [1, 1, 1, 1]], dtype=np.int64)
    i1 = np.array([[3, 3, 3, 3], [0, 1, 2, 3], [0, 1, 2, 3]], dtype=np.int64)
    ref, got = both(H, G, lambda s, a, b: type(s).scatter([a, b], [4, 4], s), src, i0, i1)
    exp = np.array([[0, 0, 0, 0.6], [2.0, 2.1, 2.2, 2.3], [1.0, 1.1, 1.2, 1.3], [0, 0, 0, 0]])
    assert np.allclose(got, exp, rtol=0, atol=1e-15)
    assert np.allclose(ref, exp, rtol=0, atol=1e-15)
    with pytest.raises(IndexError):
        type(G.ofNumpy(src)).scatter([G.ofNumpy(i0), G.ofNumpy(i1 + 1)], [4, 4], G.ofNumpy(src))


@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 4096, 4097, 100003])
def test_masked_get_1d(H, G, rng, n):
    a = rng.integers(-1000, 1000, n).astype(np.int32)
    m = a > 0
    ref, got = both(H, G, lambda a, m: a.M(m), a, m)
    assert_exact(ref, got)
    assert_exact(a[m], got)


@pytest.mark.parametrize("dt", [np.int32, np.float64])
@pytest.mark.parametrize("shift", [1, 2, 3])
def test_masked_get_and_set_on_a_shifted_view(G, rng, dt, shift):
    """The compaction's vector path on a tensor that starts at an odd element (the mask is a tensor of its own): NumPy is the checker."""
    n = 40000
    a = rng.integers(-1000, 1000, n + 8).astype(dt)
    m = rng.random(n) < 0.4
    ta, tm = G.ofNumpy(a), G.ofNumpy(m)
    assert_exact(a[shift:shift + n][m], G.toNumpy(ta[shift:shift + n].M(tm)))
    vals = rng.integers(-5, 5, int(m.sum())).astype(dt)
    want = a.copy()
    want[shift:shift + n][m] = vals
    ta[shift:shift + n].setM([tm], G.ofNumpy(vals))
    assert_exact(want, G.toNumpy(ta))


@pytest.mark.parametrize("dt", [np.float32, np.float64, np.uint8, np.bool_, np.uint16])
def test_masked_get_set_nd(H, G, rng, dt):
    a = (rng.random((37, 41)) < 0.5) if dt == np.bool_ else rng.integers(0, 100, (37, 41)).astype(dt)
    m = rng.random((37, 41)) < 0.3
    ref, got = both(H, G, lambda a, m: a.M(m), a, m)
    assert_exact(ref, got)
    assert_exact(a[m], got)
    # per-dimension masks and NoMask (Guide-Logic.md:97-100)
    m0 = rng.random(37) < 0.5
    m1 = rng.random(41) < 0.5
    for f, exp in ((lambda a, x, y: a.M(x, None), a[m0, :]), (lambda a, x, y: a.M(None, y), a[:, m1]),
                   (lambda a, x, y: a.M(x, y), a[np.ix_(m0, m1)])):
        ref, got = both(H, G, f, a, m0, m1)
        assert_exact(ref, got)
        assert_exact(exp, got)
    # masked set, also on a transposed (non-reshapeable) target
    k = int(m.sum())
    v = (rng.random(k) < 0.5) if dt == np.bool_ else rng.integers(100, 200, k).astype(dt)

    def setm(a, m, v):
        a.setM([m], v)
        return a
    ref, got = both(H, G, setm, a, m, v)
    assert_exact(ref, got)
    exp = a.copy()
    exp[m] = v
    assert_exact(exp, got)

    def setm_t(a, m, v):
        at = a.T
        at.setM([m.T.Copy()], v)
        return a
    ref, got = both(H, G, setm_t, a, m, v[: int(m.T.sum())])
    assert_exact(ref, got)


def test_mask_doc_vectors(H, G):
    a = np.array([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    m = np.array([[True, True, False], [False, False, True]])
    t = G.ofNumpy(a)
    assert G.toNumpy(t.M(G.ofNumpy(m))).tolist() == [1.0, 2.0, 6.0]                       # Guide-Logic.md:85-91
    assert G.toNumpy(t.M(G.ofNumpy(np.array([True, False])), None)).tolist() == [[1.0, 2.0, 3.0]]   # :97-100
    t.setM([G.ofNumpy(m)], G.ofNumpy(np.array([8.0, 9.0, 0.0])))
    assert G.toNumpy(t).tolist() == [[8.0, 9.0, 3.0], [4.0, 5.0, 0.0]]                    # :109-114


@pytest.mark.parametrize("shape", [(2, 4), (50,), (7, 11, 13), (3, 0), (100, 100), (16,), (4096,), (64, 48), (8, 6, 32), (1, 160, 1, 3),
                                   (333, 1024)])
def test_true_idx(H, G, rng, shape):
    m = rng.random(shape) < 0.4
    ref, got = both(H, G, lambda m: m.trueIdx(), m)
    assert_exact(ref, got)
    assert_exact(np.argwhere(m).astype(np.int64).reshape(-1, len(shape)), got)
    # all true, all false, and a target that is a column slice of a wider tensor (not dense: the general path)
    for mm in (np.ones(shape, np.bool_), np.zeros(shape, np.bool_)):
        ref, got = both(H, G, lambda m: m.trueIdx(), mm)
        assert_exact(ref, got)
    # on a permuted view
    if len(shape) == 3:
        ref, got = both(H, G, lambda m: m.permuteAxes([1, 2, 0]).trueIdx(), m)
        assert_exact(ref, got)


def test_true_idx_doc_vector(G):
    a = np.array([[True, False, True, False], [False, True, True, False]])
    assert G.toNumpy(G.ofNumpy(a).trueIdx()).tolist() == [[0, 0], [0, 2], [1, 1], [1, 2]]   # Guide-Logic.md:46-53


def test_config4_sequence_small(H, G, rng):
    """compare -> mask -> ifThenElse / countTrue / maskedGet / gather / scatter on int32, the fourth benchmark configuration."""
    n, mcount = 1 << 16, 1 << 14
    a = rng.integers(-1000, 1001, n).astype(np.int32)
    b = rng.integers(-1000, 1001, n).astype(np.int32)
    idx = rng.integers(0, n, mcount).astype(np.int64)
    idxu = rng.permutation(n)[:mcount].astype(np.int64)

    def seq(a, b, idx, idxu):
        T = type(a)
        m = a > 0
        r = T.ifThenElse(m, a, b)
        k = m.countTrue()
        g = a.M(m)
        h = T.gather([idx], a)
        s = T.scatter([idxu], [n], h)
        return m, r, k, g, h, s
    ref, got = both(H, G, seq, a, b, idx, idxu)
    for r, g in zip(ref, got):
        if isinstance(r, int):
            assert r == g == int((a > 0).sum())
        else:
            assert_exact(r, g)


@pytest.fixture(params=["two_launches", "one_pass", "tiles_do_not_wait"])
def compaction_form(request):
    """The contiguous compactions in their three forms: a counting and a moving launch (the default), one pass whose workgroups meet
    through memory (compact_one_pass = 1), and that pass with workgroups that do not poll at all: one that finds a predecessor's count
    unpublished counts the mask in front of its region itself (lookback_spins = 0: the bounded wait's way out, forced).  CountTrue
    runs in its one-launch form in the first and in the general two-pass fold in the others."""
    from deepnet_amd import native
    if request.param == "two_launches":
        yield request.param
    elif request.param == "one_pass":
        with native.option("compact_one_pass", 1), native.option("count_one_launch", 0):
            yield request.param
    else:
        with native.option("compact_one_pass", 1), native.option("lookback_spins", 0), native.option("count_one_launch", 0):
            yield request.param


@pytest.mark.parametrize("dt", [np.int32, np.float64, np.uint8, np.int16])
@pytest.mark.parametrize("n,density", [(16, 0.5), (4096, 0.5), (4112, 0.3), (1 << 20, 0.5), (3_000_016, 0.02), (3_000_016, 1.0),
                                       (3_000_016, 0.0), ((1 << 22) + 64, 0.7)])
def test_contiguous_compactions_in_every_form(G, rng, compaction_form, dt, n, density):
    """maskedGet, maskedSet, trueIdx and countTrue of contiguous 1-d data against NumPy, bit for bit, from one tile to a thousand
    tiles, all / none / few selected, twice in a row on the same stream (the second launch meets the words the first one left)."""
    a = rng.integers(0, 100, n).astype(dt)
    m = rng.random(n) < density if 0.0 < density < 1.0 else np.full(n, density == 1.0)
    ta, tm = G.ofNumpy(a), G.ofNumpy(m)
    k = int(m.sum())
    for _ in range(2):
        assert_exact(a[m], G.toNumpy(ta.M(tm)))
        assert int(tm.countTrue()) == k
        assert_exact(np.flatnonzero(m).astype(np.int64).reshape(-1, 1), G.toNumpy(tm.trueIdx()))
    vals = rng.integers(100, 200, k).astype(dt)
    want = a.copy()
    want[m] = vals
    ta.setM([tm], G.ofNumpy(vals))
    assert_exact(want, G.toNumpy(ta))
    # a 2-d mask whose elements lie in row-major order: pairs of coordinates
    if n % 16 == 0 and n >= 4096:
        m2 = m.reshape(-1, 16)
        assert_exact(np.argwhere(m2).astype(np.int64), G.toNumpy(G.ofNumpy(m2).trueIdx()))


def test_one_pass_compactions_on_two_streams(G, rng):
    """Every stream has its own tickets and tile words: compactions queued on two streams at once do not meet each other's."""
    import ctypes as C
    from deepnet_amd import native
    lib = native.load()
    native.set_option("compact_one_pass", 1)
    n = 1 << 21
    a = rng.integers(0, 1000, n).astype(np.int32)
    masks = [rng.random(n) < d for d in (0.3, 0.6)]
    streams = [C.c_void_p(), C.c_void_p()]
    for s in streams:
        native.check(lib.dnh_stream_create(C.byref(s)))
    try:
        ta = G.ofNumpy(a)
        tms = [G.ofNumpy(m) for m in masks]
        outs = [G.zeros([int(m.sum())], np.int32) for m in masks]
        native.check(lib.dnh_device_sync())
        for rep in range(4):
            for s, tm, out in zip(streams, tms, outs):
                arr = (C.POINTER(type(ta.Backend._desc(ta))) * 1)()
                dm = tm.Backend._desc(tm)
                arr[0] = C.pointer(dm)
                dt_, da = out.Backend._desc(out), ta.Backend._desc(ta)
                native.check(lib.dnh_masked_get(C.byref(dt_), C.byref(da), arr, 1, s))
        for s in streams:
            native.check(lib.dnh_stream_sync(s))
        for m, out in zip(masks, outs):
            assert_exact(a[m], G.toNumpy(out))
    finally:
        native.set_option("compact_one_pass", 0)
        for s in streams:
            native.check(lib.dnh_stream_destroy(s))
