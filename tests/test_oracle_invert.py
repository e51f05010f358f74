"""Pins the oracle's BatchedInvert (oracle/hostref.cpp href_batched_invert) without the GPU: the reference's fixture and
doc example, its singular-matrix test, closed-form inverses and the defining property A . inv(A) = I."""
import numpy as np
import pytest

from deepnet_amd.backend import SingularMatrixException
from deepnet_amd.tensor import Tensor
from invert_cases import hilbert, hilbert_inverse, inverse_error_bound, invert, kk_fixture, well_conditioned


def test_doc_example(H):
    """Tensor.fs:2820-2825: invert [[1;2];[3;4]] = [[-2;1];[1.5;-0.5]]."""
    got = invert(H, np.array([[1.0, 2.0], [3.0, 4.0]]))
    np.testing.assert_allclose(got, [[-2.0, 1.0], [1.5, -0.5]], rtol=0, atol=4e-16)


def test_reference_fixture_kk(H):
    """BaseTests.fs:214-233: Kkinv .* Kk almost equals the stacked identity with absTol = relTol = 1e-5."""
    kk, chk = kk_fixture()
    kkinv = Tensor.invert(H.ofNumpy(kk))
    ident = H.toNumpy(kkinv @ H.ofNumpy(kk))
    ids = np.broadcast_to(np.eye(10, dtype=np.float32), (3, 10, 10))
    assert np.all(np.abs(ident - ids) <= chk["abs_tol"] + chk["rel_tol"] * np.abs(ids))
    inv64 = np.linalg.inv(kk.astype(np.float64))
    assert np.abs(H.toNumpy(kkinv) - inv64).max() <= 10 * 50 * 2 ** -23 * np.abs(inv64).max()


def test_singular_matrix_raises(H):
    """BaseTests.fs:204-211."""
    with pytest.raises(SingularMatrixException):
        invert(H, np.array([[1.0, 0.0, 0.0], [1.0, 2.0, 0.0], [1.0, 0.0, 0.0]]))
    with pytest.raises(SingularMatrixException):
        invert(H, np.zeros((2, 4, 4), np.float32))


def test_closed_forms(H, rng):
    # diagonal: reciprocals, exactly
    d = rng.uniform(0.5, 8.0, 17).astype(np.float32)
    np.testing.assert_array_equal(invert(H, np.diag(d)), np.diag(np.float32(1) / d))
    # permutation matrices: the transpose, exactly (needs the row exchanges and their undoing to be right)
    perm = rng.permutation(23)
    p = np.eye(23, dtype=np.float64)[perm]
    np.testing.assert_array_equal(invert(H, p), p.T)
    # scaled permutation with a batch: exact as well
    s = rng.integers(1, 5, (4, 9)).astype(np.float64) * 2.0
    ps = np.stack([np.eye(9)[rng.permutation(9)] * s[b][:, None] for b in range(4)])
    np.testing.assert_array_equal(invert(H, ps), np.linalg.inv(ps))
    # 2x2: [[a,b],[c,d]]^-1 = [[d,-b],[-c,a]] / (ad - bc)
    m = rng.uniform(-2, 2, (50, 2, 2))
    m[:, 0, 0] += 3 * np.sign(m[:, 0, 0])
    det = m[:, 0, 0] * m[:, 1, 1] - m[:, 0, 1] * m[:, 1, 0]
    want = np.stack([np.stack([m[:, 1, 1], -m[:, 0, 1]], -1), np.stack([-m[:, 1, 0], m[:, 0, 0]], -1)], -2) / det[:, None, None]
    np.testing.assert_allclose(invert(H, m), want, rtol=1e-12, atol=1e-13)
    # Hilbert matrix, integer closed-form inverse; cond(H_6) ~ 1.5e7
    got = invert(H, hilbert(6))
    want = hilbert_inverse(6)
    assert np.abs(got - want).max() <= 6 * 2 ** -52 * 1.5e7 * np.abs(want).max()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_random_against_fp64_and_identity(H, rng, dtype):
    for shape in ((1, 1), (5, 5), (3, 40, 40), (2, 2, 65, 65)):
        a = well_conditioned(rng, shape, dtype)
        got = invert(H, a)
        inv, bound = inverse_error_bound(a)
        assert np.all(np.abs(got - inv) <= bound)
        n = shape[-1]
        assert np.abs(got.astype(np.float64) @ a.astype(np.float64) - np.eye(n)).max() <= 8 * n * np.finfo(dtype).eps * 4


def test_pivoting_is_needed_and_layouts(H, rng):
    # zero diagonal: fails without row exchanges
    a = well_conditioned(rng, (12, 12), np.float64)
    a = a[np.r_[1:12, 0]] * (1 - np.eye(12)) + np.roll(np.eye(12), 1, axis=1) * 3
    got = invert(H, a)
    np.testing.assert_allclose(got @ a, np.eye(12), atol=1e-12)
    # column-major and strided targets, broadcast source, in place
    b = well_conditioned(rng, (3, 20, 20), np.float32)
    ref = invert(H, b)
    tb = H.ofNumpy(b)
    trg = H.ofNumpy(np.zeros((3, 20, 20), np.float32)).T          # column-major matrices
    trg.FillInvert(tb)
    np.testing.assert_allclose(H.toNumpy(trg), ref, rtol=0, atol=2e-5)
    one = H.ofNumpy(b[:1])
    trg3 = H.ofNumpy(np.zeros((3, 20, 20), np.float32))
    trg3.FillInvert(one)                                          # broadcast over the batch (Tensor.fs:2814)
    got3 = H.toNumpy(trg3)
    np.testing.assert_array_equal(got3[1], got3[0])
    np.testing.assert_array_equal(got3[0], ref[0])
    tb.FillInvert(tb)                                             # in place
    np.testing.assert_array_equal(H.toNumpy(tb), ref)


def test_argument_errors(H):
    with pytest.raises(NotImplementedError):
        invert(H, np.eye(3, dtype=np.int32))
    with pytest.raises(ValueError):
        invert(H, np.ones((3, 4)))
    with pytest.raises(ValueError):
        invert(H, np.ones(4))
    assert invert(H, np.zeros((0, 3, 3))).shape == (0, 3, 3)
