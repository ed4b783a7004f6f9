"""The factorization half of the orthogonal initializer (dlmi_orthogonal_weights: host arithmetic, no device): the
weights read as a column-major matrix of max(rows, cols) x min(rows, cols), Q . sign(diag R) of its column-pivoting QR
factorization, transposed in place when rows >= cols, times the gain, written back as it lies
(v1/ops/initializers/orthogonal.cpp:132-153).  The reference takes Eigen's ColPivHouseholderQR, which is not at
hand: parity with it is unpinned.  What is pinned here: Q . sign(diag R) is fixed by the pivoting order alone, Eigen
and LAPACK's geqp3 both pick the remaining column of largest norm, and this routine agrees with scipy's (LAPACK's)
factorization to rounding, for tall, wide and square layers; and the result has orthonormal columns."""
import ctypes

import numpy as np
import pytest
import scipy.linalg

from conftest import load_package

c_sz = ctypes.c_size_t


@pytest.fixture(scope="module")
def lib():
    return load_package().load_library()


def expected(flat, rows, cols, scale):
    hi, lo = max(rows, cols), min(rows, cols)
    A = flat.reshape(lo, hi).T.astype(np.float64)  # column-major hi x lo
    Q, R, _ = scipy.linalg.qr(A, mode="economic", pivoting=True)
    W = Q * np.sign(np.diag(R))
    out = W.flatten(order="C") if rows >= cols else W.flatten(order="F")  # transposed in place, or as it lies
    return (out.astype(np.float32) * np.float32(scale)).astype(np.float32), W


@pytest.mark.parametrize("rows,cols", [(12, 5), (5, 12), (7, 7), (1, 9), (9, 1), (64, 48), (48, 64), (200, 130)])
@pytest.mark.parametrize("scale", [1.0, 1.4142135])
def test_against_lapack(lib, rows, cols, scale):
    rng = np.random.default_rng(rows * 100 + cols)
    flat = rng.standard_normal(rows * cols).astype(np.float32)
    want, W = expected(flat, rows, cols, scale)
    got = flat.copy()
    assert lib.dlmi_orthogonal_weights(c_sz(rows), c_sz(cols), ctypes.c_float(scale),
                                       got.ctypes.data_as(ctypes.c_void_p)) == 1
    assert np.max(np.abs(got - want)) < 2e-6 * scale
    lo = min(rows, cols)
    assert np.max(np.abs(W.T @ W - np.eye(lo))) < 1e-12  # what it is compared with has orthonormal columns
    hi = max(rows, cols)
    G = (got.reshape(hi, lo) if rows >= cols else got.reshape(lo, hi).T).astype(np.float64) / scale
    assert np.max(np.abs(G.T @ G - np.eye(lo))) < 1e-5


def test_dependent_columns_and_empty_layers(lib):
    """A column of zeros has no direction: it comes last in the pivoting order and stays zero (sign(0) = 0 in the
    reference's expression); an empty layer is refused."""
    rows, cols = 6, 3
    flat = np.random.default_rng(3).standard_normal(rows * cols).astype(np.float32)
    flat.reshape(cols, rows)[1, :] = 0.0  # column 1 of the 6 x 3 matrix
    got = flat.copy()
    assert lib.dlmi_orthogonal_weights(c_sz(rows), c_sz(cols), ctypes.c_float(1.0), got.ctypes.data_as(ctypes.c_void_p)) == 1
    G = got.reshape(rows, cols).astype(np.float64)
    assert np.all(G[:, 2] == 0.0)
    assert np.max(np.abs(G[:, :2].T @ G[:, :2] - np.eye(2))) < 1e-5
    assert lib.dlmi_orthogonal_weights(c_sz(0), c_sz(3), ctypes.c_float(1.0), got.ctypes.data_as(ctypes.c_void_p)) == 0
