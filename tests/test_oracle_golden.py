"""Pins the CPU oracle (oracle/oracle.cpp) against everything the reference's own tests hold for this
path: the fixture dataset/test_dataset.txt with the golden accuracy / MSE / SV-count values of
src/test/test_svc.cpp:33-37, test_svr.cpp:35-39, test_nusvc.cpp:40-44, test_nusvr.cpp:38-42,
test_oneclass_svc.cpp:27 and test_dataset.cpp:13-24, and the kernel-value oracle of
src/test/test_kernelmatrix.cpp:8-67 (restated here as an independent merge-join in Python)."""
import math
import os

import numpy as np
import pytest

import oracle_lib as O
from thundersvm_amd.data import load_libsvm

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "test_dataset.txt")


@pytest.fixture(scope="module")
def data():
    return load_libsvm(FIXTURE)


def test_fixture_shape(data):      # test_dataset.cpp:13-24
    assert data.n == 150 and data.n_features == 4
    labels, counts = [], []
    for v in data.y:
        if v not in labels:
            labels.append(v)
            counts.append(0)
        counts[labels.index(v)] += 1
    assert labels == [0, 2, 3] and counts == [49, 50, 51]


@pytest.mark.parametrize("mode", [0, 1])
def test_golden_models(data, mode):
    d = data
    m = O.Model(d.ptr, d.col, d.val, d.y, O.make_param(O.C_SVC, O.RBF, gamma=0.5, C_=100, expf_mode=mode))
    pred, _ = m.predict(d.ptr, d.col, d.val, 100)
    assert abs((pred == d.y).mean() - 0.98) < 1e-5
    assert list(m.label) == [0, 2, 3]
    m = O.Model(d.ptr, d.col, d.val, d.y, O.make_param(O.EPSILON_SVR, O.RBF, gamma=0.5, C_=100, expf_mode=mode))
    pred, _ = m.predict(d.ptr, d.col, d.val, 100)
    assert abs(((pred - d.y) ** 2).mean() - 0.020752) < 1e-3
    m = O.Model(d.ptr, d.col, d.val, d.y, O.make_param(O.NU_SVC, O.RBF, gamma=0.5, nu=0.1, C_=100, expf_mode=mode))
    pred, _ = m.predict(d.ptr, d.col, d.val, 100)
    assert abs((pred == d.y).mean() - 0.98) < 1e-3
    m = O.Model(d.ptr, d.col, d.val, d.y, O.make_param(O.NU_SVR, O.RBF, gamma=0.5, nu=0.1, C_=100, expf_mode=mode))
    pred, _ = m.predict(d.ptr, d.col, d.val, 100)
    assert abs(((pred - d.y) ** 2).mean() - 0.028369) < 1.2e-5
    m = O.Model(d.ptr, d.col, d.val, d.y, O.make_param(O.ONE_CLASS, O.RBF, gamma=0.5, nu=0.1, expf_mode=mode))
    pred, _ = m.predict(d.ptr, d.col, d.val, 100)
    assert int((pred > 0).sum()) == 135


def _rows(d):
    return [dict(zip(d.col[d.ptr[i]:d.ptr[i + 1]].tolist(), d.val[d.ptr[i]:d.ptr[i + 1]].tolist())) for i in range(d.n)]


def _ref_kernel(rows, x, y, kt, gamma, coef0, degree):
    """test_kernelmatrix.cpp:8-67: sparse merge-join dot / squared distance, float transcendental."""
    a, b = rows[x], rows[y]
    if kt == O.RBF:
        keys = set(a) | set(b)
        s = sum((a.get(k, 0.0) - b.get(k, 0.0)) ** 2 for k in sorted(keys))
        return float(np.float32(math.exp(np.float32(-gamma * s))))
    dot = sum(a[k] * b[k] for k in sorted(a) if k in b)
    if kt == O.POLY:
        return float(np.float32(np.float32(gamma * dot + coef0) ** np.float32(degree)))
    if kt == O.SIGMOID:
        return float(np.float32(math.tanh(np.float32(gamma * dot + coef0))))
    return dot


@pytest.mark.parametrize("kt,prm", [(O.RBF, dict(gamma=0.5)), (O.POLY, dict(gamma=0.5, degree=3, coef0=0.1)),
                                    (O.LINEAR, dict()), (O.SIGMOID, dict(gamma=0.5, coef0=0.1))])
@pytest.mark.parametrize("mode", [0, 1])
def test_kernel_values(data, kt, prm, mode):
    d = data
    km = O.KernelMatrix(d.ptr, d.col, d.val, O.make_param(kernel_type=kt, expf_mode=mode, **prm))
    rows = _rows(d)
    g, c0, dg = prm.get("gamma", 0.0), prm.get("coef0", 0.0), prm.get("degree", 3)
    assert km.n_features == 5          # largest feature id + 1 (kernelmatrix.cpp:200-206)
    diag = km.diag()
    for i in range(d.n):
        assert abs(diag[i] - _ref_kernel(rows, i, i, kt, g, c0, dg)) < 1e-4
    idx = np.arange(10) * 3 + 4        # test_kernelmatrix.cpp:83-86
    k = km.get_rows(idx)
    want = np.array([[_ref_kernel(rows, i, j, kt, g, c0, dg) for j in range(d.n)] for i in idx])
    assert np.abs(k - want).max() < 1e-4          # the reference's own tolerance
    assert np.abs(k - want).max() < 2e-6          # and what the arithmetic actually allows
    batch = d.rows(np.arange(10))
    k2 = km.get_rows_instances(batch.ptr, batch.col, batch.val)
    want2 = np.array([[_ref_kernel(rows, i, j, kt, g, c0, dg) for j in range(d.n)] for i in range(10)])
    assert np.abs(k2 - want2).max() < 2e-6


def test_kernel_values_vs_sklearn(data):
    from sklearn.metrics.pairwise import linear_kernel, polynomial_kernel, rbf_kernel, sigmoid_kernel
    d = data
    x = d.to_dense()[:, 1:]
    idx = np.arange(0, 150, 7)
    for kt, prm, ref in [(O.RBF, dict(gamma=0.5), rbf_kernel(x[idx], x, gamma=0.5)),
                         (O.LINEAR, dict(), linear_kernel(x[idx], x)),
                         (O.POLY, dict(gamma=0.5, degree=3, coef0=0.1), polynomial_kernel(x[idx], x, degree=3, gamma=0.5, coef0=0.1)),
                         (O.SIGMOID, dict(gamma=0.5, coef0=0.1), sigmoid_kernel(x[idx], x, gamma=0.5, coef0=0.1))]:
        km = O.KernelMatrix(d.ptr, d.col, d.val, O.make_param(kernel_type=kt, **prm))
        assert np.abs(km.get_rows(idx) - ref).max() < 2e-6


def test_out_of_range_test_features():
    """kernelmatrix.cpp:290-295,392: dropped from the dot product, kept in the self dot."""
    ptr, col, val = [0, 2, 3], [1, 2, 1], [1.0, 2.0, 3.0]
    km = O.KernelMatrix(ptr, col, val, O.make_param(kernel_type=O.RBF, gamma=0.25, expf_mode=0))
    k = km.get_rows_instances([0, 3], [1, 2, 7], [1.0, 1.0, 5.0])
    sd_t = 1 + 1 + 25
    want0 = np.float32(math.exp(np.float32(-(sd_t + 5.0 - 2 * 3.0) * 0.25)))
    want1 = np.float32(math.exp(np.float32(-(sd_t + 9.0 - 2 * 3.0) * 0.25)))
    assert k[0, 0] == want0 and k[0, 1] == want1
    lin = O.KernelMatrix(ptr, col, val, O.make_param(kernel_type=O.LINEAR))
    assert np.array_equal(lin.get_rows_instances([0, 3], [1, 2, 7], [1.0, 1.0, 5.0]), [[3.0, 3.0]])


def test_against_libsvm_solver(data):
    """sklearn's SVC is LibSVM: a different solver reaches the same optimum to ~1e-3 (paper Table 4)."""
    from sklearn.svm import SVC
    d = data
    sel = np.flatnonzero(d.y != 3)
    sub = d.rows(sel)
    x = sub.to_dense()[:, 1:]
    sk = SVC(C=100, gamma=0.5, tol=1e-5).fit(x, sub.y)
    m = O.Model(sub.ptr, sub.col, sub.val, sub.y, O.make_param(O.C_SVC, O.RBF, gamma=0.5, C_=100))
    _, dec = m.predict(sub.ptr, sub.col, sub.val)
    # LibSVM's decision function is positive for classes_[1]; ours for the first label seen (0)
    sk_dec = sk.decision_function(x)
    assert np.abs(np.abs(dec[:, 0]) - np.abs(sk_dec)).max() < 5e-2
    assert abs(abs(m.rho[0]) - abs(sk.intercept_[0])) < 5e-2
    assert np.array_equal(np.sign(dec[:, 0]), -np.sign(sk_dec))
