"""Inputs and checks shared by the CPU (oracle) and GPU tests of BatchedInvert."""
import json
import os

import numpy as np

from deepnet_amd.tensor import Tensor

HERE = os.path.dirname(os.path.abspath(__file__))


def kk_fixture():
    """The reference's own test matrix stack (Tensor.Test/TestData/MatInv.h5 "Kk", single, [3; 10; 10])."""
    j = json.load(open(os.path.join(HERE, "golden", "matinv_kk.json")))
    return np.frombuffer(bytes.fromhex(j["data_hex"]), "<f4").reshape(j["shape"]).copy(), j["check"]


def hilbert(n):
    i = np.arange(1, n + 1, dtype=np.float64)
    return 1.0 / (i[:, None] + i[None, :] - 1.0)


def hilbert_inverse(n):
    """Closed form: (-1)^(i+j) (i+j-1) C(n+i-1, n-j) C(n+j-1, n-i) C(i+j-2, i-1)^2, all integers."""
    from math import comb
    out = np.empty((n, n), dtype=np.float64)
    for i in range(1, n + 1):
        for j in range(1, n + 1):
            out[i - 1, j - 1] = (-1) ** (i + j) * (i + j - 1) * comb(n + i - 1, n - j) * comb(n + j - 1, n - i) * comb(i + j - 2, i - 1) ** 2
    return out


def well_conditioned(rng, shape, dtype):
    """Random matrices with singular values in [1, 4] (condition number <= 4) and no structure that avoids pivoting."""
    *batch, n, _ = shape
    out = np.empty(shape, dtype=np.float64)
    for idx in np.ndindex(*batch):
        q1, _ = np.linalg.qr(rng.standard_normal((n, n)))
        q2, _ = np.linalg.qr(rng.standard_normal((n, n)))
        out[idx] = (q1 * rng.uniform(1.0, 4.0, n)) @ q2
    return out.astype(dtype)


def invert(mod, a):
    return mod.toNumpy(Tensor.invert(mod.ofNumpy(a)))


def inverse_error_bound(a, factor=8.0):
    """|computed - exact| <= factor * n * eps * cond(A) * max|inv(A)| per matrix (first-order bound for LU/Gauss-Jordan with
    partial pivoting; the growth factor is absorbed into `factor` for these well-conditioned inputs)."""
    a64 = a.astype(np.float64)
    n = a.shape[-1]
    inv = np.linalg.inv(a64)
    eps = np.finfo(a.dtype).eps
    cond = np.linalg.cond(a64)
    return inv, factor * n * eps * cond[..., None, None] * np.abs(inv).max(axis=(-1, -2), keepdims=True)
