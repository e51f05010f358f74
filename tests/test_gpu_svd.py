"""GPU parity: BatchedSVD, SymmetricEigenDecomposition and pseudoInvert through the C ABI against the oracle (numpy's LAPACK gesdd /
syevd, the routines the reference's host backend calls, Host/HostBackend.fs:579-628).  Singular vectors and eigenvectors are defined
up to sign (and up to rotation inside repeated values), so vectors are compared through what defines them: reconstruction,
orthogonality and the residual A v - lambda v; values are compared with the oracle's to tol * largest value, tol = 50 * max(M, N) * eps."""
import numpy as np
import pytest

from util import both

pytestmark = pytest.mark.gpu


def tol_of(dt, n):
    return 50 * max(n, 1) * np.finfo(dt).eps


def check_svd(a, u, s, v, s_ref):
    m, n = a.shape[-2:]
    k = min(m, n)
    t = tol_of(a.dtype, max(m, n))
    a64, u64, s64, v64 = (x.astype(np.float64) for x in (a, u, s, v))
    scale = max(float(np.abs(s_ref).max(initial=0.0)), np.finfo(a.dtype).tiny)
    assert s.shape == s_ref.shape and np.all(s64[..., :-1] >= s64[..., 1:]) and np.all(s64 >= 0)
    assert np.abs(s64 - s_ref.astype(np.float64)).max(initial=0.0) <= t * scale
    recon = (u64[..., :, :k] * s64[..., None, :]) @ np.swapaxes(v64[..., :, :k], -1, -2)
    assert np.abs(recon - a64).max(initial=0.0) <= t * scale
    assert np.abs(np.swapaxes(u64, -1, -2) @ u64 - np.eye(m)).max(initial=0.0) <= t
    assert np.abs(np.swapaxes(v64, -1, -2) @ v64 - np.eye(n)).max(initial=0.0) <= t


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(4, 4), (5, 3), (3, 5), (1, 1), (1, 6), (7, 1), (3, 10, 10), (2, 3, 7, 4), (64, 64), (130, 70), (33, 257)])
def test_svd(H, G, rng, dt, shape):
    a = rng.standard_normal(shape).astype(dt)
    f = lambda x: type(x).SVD(x)
    (ur, sr, vr), (u, s, v) = both(H, G, f, a)
    check_svd(a, u, s, v, sr)
    check_svd(a, ur, sr, vr, sr)          # the oracle meets the same contract
    ref, got = both(H, G, lambda x: type(x).SVDWithoutUV(x), a)
    assert np.abs(got.astype(np.float64) - ref).max() <= tol_of(dt, max(shape[-2:])) * np.abs(ref).max()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_svd_rank_deficient_zero_and_views(H, G, rng, dt):
    b = rng.standard_normal((9, 3)).astype(dt)
    low = (b @ b.T).astype(dt)                                   # 9 x 9, rank 3: six vectors come from the complement
    dup = np.concatenate([b, b[:, :2]], axis=1).astype(dt)       # 9 x 5 with repeated columns
    for a in (low, dup, np.zeros((4, 6), dt), np.eye(5, dtype=dt), np.diag(np.array([3, 3, 3, 1], dt))):
        (ur, sr, vr), (u, s, v) = both(H, G, lambda x: type(x).SVD(x), a)
        check_svd(a, u, s, v, sr)
    # transposed and strided source views, targets of the frontend's mixed orders
    big = rng.standard_normal((3, 12, 16)).astype(dt)
    f = lambda x: type(x).SVD(x.T[:, 2:11, 1:9])                # [3; 9; 8] view of the transposed matrices
    (ur, sr, vr), (u, s, v) = both(H, G, f, big)
    check_svd(np.swapaxes(big, -1, -2)[:, 2:11, 1:9], u, s, v, sr)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_pseudo_invert(H, G, dt):
    """Tensor.Test/BaseTests.fs:234-257: pinv(pinv(A)) = A for a random 4 x 4 matrix, and the singular 3 x 3 example."""
    rng = np.random.default_rng(123)
    dm = rng.uniform(-1, 1, (4, 4)).astype(dt)
    rc = 1e-6 if dt == np.float32 else 1e-15
    ref, got = both(H, G, lambda x: type(x).pseudoInvert(x, rc), dm)
    t = tol_of(dt, 4) * np.linalg.cond(dm.astype(np.float64))
    assert np.abs(got - ref).max() <= t * np.abs(ref).max()
    ref2, got2 = both(H, G, lambda x: type(x).pseudoInvert(type(x).pseudoInvert(x, rc), rc), dm)
    assert np.allclose(got2, dm, rtol=0, atol=t * 10)
    sing = np.array([[1.0, 0.0, 0.0], [1.0, 2.0, 0.0], [1.0, 0.0, 0.0]], dt)
    ref, got = both(H, G, lambda x: type(x).pseudoInvert(x, 1e-5 if dt == np.float32 else 1e-12), sing)
    assert np.allclose(got, np.linalg.pinv(sing.astype(np.float64)), atol=1e-5 if dt == np.float32 else 1e-12)
    assert np.allclose(ref, got, atol=1e-5 if dt == np.float32 else 1e-12)
    batch = rng.uniform(-1, 1, (3, 5, 5)).astype(dt)
    ref, got = both(H, G, lambda x: type(x).pseudoInvert(x, rc), batch)
    assert np.allclose(got, np.linalg.inv(batch.astype(np.float64)), rtol=0, atol=tol_of(dt, 5) * 1e3)


def check_eig(sym, w, v, w_ref):
    n = sym.shape[0]
    t = tol_of(sym.dtype, n)
    s64, w64, v64 = sym.astype(np.float64), w.astype(np.float64), v.astype(np.float64)
    scale = max(float(np.abs(s64).max(initial=0.0)) * n ** 0.5, np.finfo(sym.dtype).tiny)
    assert np.all(w64[:-1] <= w64[1:])
    assert np.abs(w64 - w_ref.astype(np.float64)).max(initial=0.0) <= t * scale
    assert np.abs(s64 @ v64 - v64 * w64).max(initial=0.0) <= t * scale
    assert np.abs(v64.T @ v64 - np.eye(n)).max(initial=0.0) <= t


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("n", [1, 2, 5, 64, 131])
@pytest.mark.parametrize("part", ["Upper", "Lower"])
def test_symmetric_eig(H, G, rng, dt, n, part):
    b = rng.standard_normal((n, n)).astype(dt)
    sym = ((b + b.T) / 2).astype(dt)
    # the other triangle holds values that must be ignored
    junk = sym.copy()
    if part == "Upper":
        junk[np.tril_indices(n, -1)] = 777
    else:
        junk[np.triu_indices(n, 1)] = -777
    f = lambda x: type(x).symmetricEigenDecomposition(part, x)
    (wr, vr), (w, v) = both(H, G, f, junk)
    check_eig(sym, w, v, wr)
    check_eig(sym, wr, vr, wr)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_symmetric_eig_special_spectra(H, G, dt):
    cases = [np.array([[0, 1], [1, 0]], dt),                        # eigenvalues -1, +1: equal magnitudes of opposite sign
             np.eye(4, dtype=dt) * 2,                               # one eigenvalue, four times
             np.zeros((3, 3), dt),
             np.diag(np.array([-5, 5, 1e-3, 0], dt)),
             np.array([[2, -1, 0], [-1, 2, -1], [0, -1, 2]], dt)]   # 2 - sqrt 2, 2, 2 + sqrt 2
    for sym in cases:
        (wr, vr), (w, v) = both(H, G, lambda x: type(x).symmetricEigenDecomposition("Upper", x), sym)
        check_eig(sym, w, v, wr)
    w = both(H, G, lambda x: type(x).symmetricEigenDecomposition("Lower", x)[0], cases[-1])[1]
    assert np.allclose(w, [2 - 2 ** 0.5, 2, 2 + 2 ** 0.5], atol=1e-5)


def test_decompositions_need_floating_point_and_matrices(G):
    T = type(G.zeros([1], np.float32))
    with pytest.raises(NotImplementedError):
        T.SVD(G.ofNumpy(np.ones((3, 3), np.int32)))
    with pytest.raises(NotImplementedError):
        T.symmetricEigenDecomposition("Upper", G.ofNumpy(np.ones((3, 3), np.int64)))
    with pytest.raises(ValueError):
        T.SVD(G.ofNumpy(np.ones(3, np.float32)))
    with pytest.raises(ValueError):
        T.symmetricEigenDecomposition("Upper", G.ofNumpy(np.ones((2, 3), np.float32)))
    with pytest.raises(ValueError):
        T.pseudoInvert(G.ofNumpy(np.ones((5, 3), np.float32)))     # the reference's pseudoInvert only takes square matrices


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(3, 96, 80), (1030, 200), (200, 1030), (2, 257, 129)])
def test_svd_block_rounds(H, G, rng, dt, shape):
    """64 columns and more take the block rounds: batches, several pieces of the rows, a last block of fewer than 16 columns, an odd
    number of blocks, row counts that are not multiples of 4."""
    a = rng.standard_normal(shape).astype(dt)
    (ur, sr, vr), (u, s, v) = both(H, G, lambda x: type(x).SVD(x), a)
    check_svd(a, u, s, v, sr)
    ref, got = both(H, G, lambda x: type(x).SVDWithoutUV(x), a)
    assert np.abs(got.astype(np.float64) - ref).max() <= tol_of(dt, max(shape[-2:])) * np.abs(ref).max()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_svd_block_rounds_rank_deficient_and_graded(H, G, rng, dt):
    low = (rng.standard_normal((300, 40)) @ rng.standard_normal((40, 100))).astype(dt)          # rank 40 of 100
    graded = (rng.standard_normal((150, 90)) * np.logspace(0, -5 if dt == np.float32 else -12, 90)).astype(dt)
    for a in (low, graded, np.zeros((70, 70), dt), np.eye(80, dtype=dt)):
        (ur, sr, vr), (u, s, v) = both(H, G, lambda x: type(x).SVD(x), a)
        check_svd(a, u, s, v, sr)


@pytest.mark.parametrize("dt,scale", [(np.float32, 1e-25), (np.float32, 1e25), (np.float64, 1e-170), (np.float64, 1e170)])
@pytest.mark.parametrize("n", [6, 80])
def test_extreme_magnitudes(H, G, rng, dt, scale, n):
    """Entries whose squares leave the element type's range: the work matrix is scaled by a power of two first."""
    a = (rng.standard_normal((n + 3, n)) * scale).astype(dt)
    (ur, sr, vr), (u, s, v) = both(H, G, lambda x: type(x).SVD(x), a)
    assert np.all(np.isfinite(s)) and s[0] > 0
    check_svd(a, u, s, v, sr)
    b = rng.standard_normal((n, n))
    sym = ((b + b.T) / 2 * scale).astype(dt)
    (wr, vr2), (w, v2) = both(H, G, lambda x: type(x).symmetricEigenDecomposition("Upper", x), sym)
    assert np.all(np.isfinite(w)) and np.abs(w).max() > 0
    check_eig(sym, w, v2, wr)


def test_svd_more_matrices_than_one_launch_takes(H, G, rng):
    """70000 matrices: the sweeps run on slices of at most 65535 matrices."""
    a = rng.standard_normal((70000, 3, 2)).astype(np.float32)
    u, s, v = (G.toNumpy(t) for t in type(G.ofNumpy(a)).SVD(G.ofNumpy(a)))
    ref = np.linalg.svd(a.astype(np.float64), compute_uv=False)
    assert np.abs(s - ref).max() <= 1e-5 * ref.max()
    recon = (u[..., :, :2] * s[..., None, :]) @ np.swapaxes(v, -1, -2)
    assert np.abs(recon - a).max() <= 1e-5 * ref.max()
