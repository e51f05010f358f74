"""BatchedInvert on the GPU (blocked Gauss-Jordan with partial pivoting + MFMA update) through the C ABI, against the
oracle's LAPACK-style LU inversion, the reference's fixture and closed forms.  Both sides are backward-stable algorithms with
different operation orders, so parity is stated as a bound: |gpu - exact| and |oracle - exact| <= 8 n eps cond(A) max|inv(A)|."""
import numpy as np
import pytest

from deepnet_amd.backend import SingularMatrixException
from deepnet_amd.tensor import Tensor
from invert_cases import hilbert, hilbert_inverse, inverse_error_bound, invert, kk_fixture, well_conditioned

pytestmark = pytest.mark.gpu


@pytest.fixture(params=[0, 1], ids=["column_by_column", "tournament"])
def pivot_form(request):
    """Runs a test once with every panel eliminated column by column in one workgroup and once with the panels' pivots found by
    tournament, whatever the size (the library's own choice: the tournament from 33 rows on)."""
    from deepnet_amd import native
    with native.option("invert_tournament", request.param):
        yield request.param


def test_doc_example_and_fixture(H, G, pivot_form):
    got = invert(G, np.array([[1.0, 2.0], [3.0, 4.0]]))
    np.testing.assert_allclose(got, [[-2.0, 1.0], [1.5, -0.5]], rtol=0, atol=2e-15)   # cond = 15, a few ulp
    kk, chk = kk_fixture()
    kkinv = Tensor.invert(G.ofNumpy(kk))
    ident = G.toNumpy(kkinv @ G.ofNumpy(kk))
    ids = np.broadcast_to(np.eye(10, dtype=np.float32), (3, 10, 10))
    assert np.all(np.abs(ident - ids) <= chk["abs_tol"] + chk["rel_tol"] * np.abs(ids))       # BaseTests.fs:214-233
    ref = invert(H, kk)
    assert np.abs(G.toNumpy(kkinv) - ref).max() <= 20 * 50 * 2 ** -23 * np.abs(ref).max()


def test_singular_matrix_raises(G, pivot_form):
    with pytest.raises(SingularMatrixException):
        invert(G, np.array([[1.0, 0.0, 0.0], [1.0, 2.0, 0.0], [1.0, 0.0, 0.0]]))               # BaseTests.fs:204-211
    with pytest.raises(SingularMatrixException):
        invert(G, np.zeros((2, 40, 40), np.float32))
    # the flag does not stick: the next call succeeds
    np.testing.assert_array_equal(invert(G, np.eye(5)), np.eye(5))


def test_exact_cases(G, rng, pivot_form):
    d = rng.uniform(0.5, 8.0, 70).astype(np.float32)
    np.testing.assert_array_equal(invert(G, np.diag(d)), np.diag(np.float32(1) / d))
    for n in (23, 64, 100):
        p = np.eye(n, dtype=np.float64)[rng.permutation(n)]
        np.testing.assert_array_equal(invert(G, p), p.T)
    s = rng.integers(1, 5, (4, 45)).astype(np.float32) * 2
    ps = np.stack([np.eye(45, dtype=np.float32)[rng.permutation(45)] * s[b][:, None] for b in range(4)])
    np.testing.assert_array_equal(invert(G, ps), np.linalg.inv(ps.astype(np.float64)).astype(np.float32))
    got = invert(G, hilbert(6))
    want = hilbert_inverse(6)
    assert np.abs(got - want).max() <= 6 * 2 ** -52 * 1.5e7 * np.abs(want).max()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(1, 1), (2, 2), (31, 31), (32, 32), (33, 33), (3, 64, 64), (2, 3, 50, 50), (130, 130), (257, 257), (2, 500, 500),
                                   (2, 600, 600), (1100, 1100)])   # more rows than the tournament's last round takes: two rounds
def test_against_oracle_and_fp64(H, G, rng, dtype, shape, pivot_form):
    a = well_conditioned(rng, shape, dtype)
    got = invert(G, a)
    ref = invert(H, a)
    inv, bound = inverse_error_bound(a)
    assert got.dtype == ref.dtype and got.shape == ref.shape
    assert np.all(np.abs(got - inv) <= bound), float((np.abs(got - inv) / bound).max())
    assert np.all(np.abs(ref - inv) <= bound)
    assert np.all(np.abs(got.astype(np.float64) - ref.astype(np.float64)) <= 2 * bound)


def test_pivoting_layouts_inplace_broadcast(H, G, rng, pivot_form):
    a = well_conditioned(rng, (70, 70), np.float64)
    a = a * (1 - np.eye(70)) + np.roll(np.eye(70), 1, axis=1) * 3            # zero diagonal
    got = invert(G, a)
    np.testing.assert_allclose(got @ a, np.eye(70), atol=1e-10)
    b = well_conditioned(rng, (3, 45, 45), np.float32)
    ref = invert(G, b)
    tb = G.ofNumpy(b)
    trg = G.ofNumpy(np.zeros((3, 45, 45), np.float32)).T                      # column-major target
    trg.FillInvert(tb)
    np.testing.assert_array_equal(G.toNumpy(trg), ref)
    src_t = G.ofNumpy(np.ascontiguousarray(b.transpose(0, 2, 1))).T           # column-major source
    np.testing.assert_array_equal(G.toNumpy(Tensor.invert(src_t)), ref)
    trg3 = G.ofNumpy(np.zeros((3, 45, 45), np.float32))
    trg3.FillInvert(G.ofNumpy(b[:1]))                                         # broadcast batch (stride 0)
    got3 = G.toNumpy(trg3)
    np.testing.assert_array_equal(got3[2], got3[0])
    np.testing.assert_array_equal(got3[0], ref[0])
    tb.FillInvert(tb)                                                         # in place
    np.testing.assert_array_equal(G.toNumpy(tb), ref)
    sl = G.ofNumpy(np.zeros((3, 50, 60), np.float32))[:, 2:47, 5:50]          # sliced target
    sl.FillInvert(G.ofNumpy(b))
    np.testing.assert_array_equal(G.toNumpy(sl), ref)


def test_argument_errors(G):
    with pytest.raises(NotImplementedError):
        invert(G, np.eye(3, dtype=np.int32))
    with pytest.raises(ValueError):
        invert(G, np.ones((3, 4)))
    with pytest.raises(ValueError):
        invert(G, np.ones(4))
    assert invert(G, np.zeros((0, 3, 3))).shape == (0, 3, 3)


def test_large_matrix_by_identity(G, rng, pivot_form):
    """1000 x 1000 single (a size of the reference's benchmark): inv(A) . A = I within n eps cond."""
    n = 1000
    a = (rng.standard_normal((n, n)) / np.sqrt(n) + 2 * np.eye(n)).astype(np.float32)
    ta = G.ofNumpy(a)
    prod = G.toNumpy(Tensor.invert(ta) @ ta)
    assert np.abs(prod - np.eye(n)).max() <= 8 * n * 2 ** -23 * np.linalg.cond(a.astype(np.float64))


def test_two_rounds_of_games(G, rng):
    """4400 rows: the first panels have more rows than 16 x 256, so a round of games leaves more than 512 candidates and a second round
    runs before the last workgroup's; the pivots must still be good ones (no diagonal dominance to lean on)."""
    n = 4400
    q, _ = np.linalg.qr(rng.standard_normal((n, n)))
    a = (q * rng.uniform(1.0, 4.0, n)).astype(np.float32)          # orthogonal columns scaled: condition number 4, no structure
    ta = G.ofNumpy(a)
    prod = G.toNumpy(Tensor.invert(ta) @ ta)
    assert np.abs(prod - np.eye(n)).max() <= 8 * n * 2 ** -23 * 4


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_tournament_pivots(G, rng, dtype):
    """What the tournament has to get right beyond accuracy on friendly matrices: a panel whose large entries sit in few rows (every
    workgroup of the first round must hand on more than its first choice), an entry that
    dwarfs its column, and a singular matrix with a column of zeros."""
    from deepnet_amd import native
    n = 700
    with native.option("invert_tournament", 1):
        a = well_conditioned(rng, (n, n), dtype).astype(np.float64)
        a[300:340] *= 1e3                                   # forty rows carry every column's largest entries
        a[17, 5] = 1e6
        a = a.astype(dtype)
        got = invert(G, a)
        inv, bound = inverse_error_bound(a, factor=32.0)
        assert np.all(np.abs(got - inv) <= bound), float((np.abs(got - inv) / bound).max())
        z = a.copy()
        z[:, 40] = 0
        with pytest.raises(SingularMatrixException):
            invert(G, z)
        # the games are deterministic: the same bits every time
        np.testing.assert_array_equal(invert(G, a), got)


def test_large_scaled_permutation_is_exact(G, rng):
    """12 320 rows: the panel's tournament takes two rounds of games before the last, and the permutation that undoes the row
    exchanges no longer fits the LDS of the kernel that composes it.  A permutation matrix with rows scaled by powers of two has an
    inverse that every step computes exactly: its transpose with the reciprocal scales."""
    n = 12320
    perm = rng.permutation(n)
    scale = np.ldexp(1.0, rng.integers(-3, 4, n)).astype(np.float32)
    a = np.zeros((n, n), np.float32)
    a[np.arange(n), perm] = scale                       # row i holds scale[i] in column perm[i]
    got = invert(G, a)
    rows, cols = np.nonzero(got)
    assert rows.size == n
    assert np.array_equal(rows[np.argsort(rows)], np.arange(n))
    want = np.zeros(n, np.float32)
    want[perm] = np.float32(1) / scale                  # inverse: row perm[i] holds 1 / scale[i] in column i
    order = np.argsort(rows)
    assert np.array_equal(cols[order], np.argsort(perm))
    assert np.array_equal(got[rows[order], cols[order]], want)
