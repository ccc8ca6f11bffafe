"""Prediction in one pass (tsvm_predict_dec_values_dense behind SvmModel::predict_dec_values, replacing
svmmodel.cpp:74-117's get_rows + sum_kernel_values): decision values against the CPU oracle's serial sums at the
path's tolerance (1e-6 absolute), and against the two-call form on the device, for every shape the kernels
distinguish: one to eleven coefficient rows, few / many features, indicator columns, all four kernels, batch sizes
that do and do not fill a tile, rows already resident on the device."""
import numpy as np
import pytest

import oracle_lib as O
from thundersvm_amd import data as D
from thundersvm_amd.model import Dataset, Model, make_param

pytestmark = pytest.mark.gpu


def _oparam(prm):
    return O.make_param(svm_type=prm.svm_type, kernel_type=prm.kernel_type, degree=prm.degree, gamma=prm.gamma,
                        coef0=prm.coef0, C_=prm.C, nu=prm.nu, p=prm.p, epsilon=prm.epsilon, max_iter=prm.max_iter,
                        max_mem_size=prm.max_mem_size, expf_mode=1)


def _blobs(rng, k, per, d, one_hot=0, spread=0.8):
    """k Gaussian classes in d continuous features, optionally followed by a `one_hot`-way indicator block."""
    centres = 2.0 * rng.standard_normal((k, d))
    cls = rng.permutation(np.repeat(np.arange(k), per))
    x = (centres[cls] + spread * rng.standard_normal((k * per, d))).astype(np.float32)
    if one_hot:
        hot = np.zeros((k * per, one_hot), dtype=np.float32)
        hot[np.arange(k * per), (cls * 3 + rng.integers(0, 3, k * per)) % one_hot] = 1.0
        x = np.concatenate([x, hot], axis=1)
    return x, (cls + 1).astype(np.float64)


def _check(tr, te, prm, monkeypatch, batch=-1, tol=1e-6):
    gm = Model(prm.svm_type).train(tr, prm)
    om = O.Model(tr.ptr, tr.col, tr.val, tr.y, _oparam(prm))
    assert gm.total_sv == om.total_sv
    glab, gdec = gm.predict(te, batch)
    olab, odec = om.predict(te.ptr, te.col, te.val, 100)
    scale = max(1.0, float(np.abs(gm.coef).sum()) * 1e-6)      # (huge cancelling coefficients move with the order of the sums)
    assert np.abs(gdec - odec).max() < tol * scale
    clear = np.abs(odec).min(axis=1) > tol * scale
    if prm.svm_type in (0, 1):
        assert np.array_equal(glab[clear], olab[clear])
    # the same model through the two-call form (kernel rows written out, then sum_kernel_values)
    monkeypatch.setenv("TSVM_PREDICT_UNFUSED", "1")
    _, tdec = gm.predict(te, 100)
    monkeypatch.delenv("TSVM_PREDICT_UNFUSED")
    assert np.abs(gdec - tdec).max() < 1e-9 * max(1.0, float(np.abs(gm.coef).sum()))
    # rows resident on the device give what rows from the host give
    ds = Dataset(te).to_device()
    _, ddec = gm.predict(ds, batch)
    assert np.abs(ddec - gdec).max() < 1e-9 * max(1.0, float(np.abs(gm.coef).sum()))
    return gm, gdec


@pytest.mark.parametrize("k", [2, 3, 4, 5, 6, 7, 8, 9, 10, 12])
def test_class_counts_few_features(k, monkeypatch):
    rng = np.random.default_rng(100 + k)
    x, y = _blobs(rng, k, 60, 7)
    xt, _ = _blobs(np.random.default_rng(200 + k), k, 13, 7)
    _check(D.from_dense(x, y), D.from_dense(xt, np.zeros(len(xt))), make_param(svm_type=0, kernel_type=2, gamma=0.3, C=4.0),
           monkeypatch)


@pytest.mark.parametrize("k", [2, 3, 7, 9, 12])
def test_class_counts_indicator_columns(k, monkeypatch):
    rng = np.random.default_rng(300 + k)
    x, y = _blobs(rng, k, 80, 5, one_hot=40)
    xt, _ = _blobs(np.random.default_rng(400 + k), k, 21, 5, one_hot=40)
    gm, _ = _check(D.from_dense(x, y), D.from_dense(xt, np.zeros(len(xt))),
                   make_param(svm_type=0, kernel_type=2, gamma=0.2, C=4.0), monkeypatch)
    # a batch whose values in those columns are not all zeros and ones takes the plain columns
    xt2 = xt.copy()
    xt2[3, -2] = 0.5
    te2 = D.from_dense(xt2, np.zeros(len(xt2)))
    om = O.Model(D.from_dense(x, y).ptr, D.from_dense(x, y).col, D.from_dense(x, y).val, y, _oparam(make_param(svm_type=0, kernel_type=2, gamma=0.2, C=4.0)))
    _, gdec = gm.predict(te2)
    _, odec = om.predict(te2.ptr, te2.col, te2.val, 100)
    assert np.abs(gdec - odec).max() < 1e-6


@pytest.mark.parametrize("k", [2, 4, 12, 26])
def test_class_counts_many_features(k, monkeypatch):
    rng = np.random.default_rng(500 + k)
    x, y = _blobs(rng, k, 40, 200, spread=1.5)
    xt, _ = _blobs(np.random.default_rng(600 + k), k, 9, 200, spread=1.5)
    _check(D.from_dense(x, y), D.from_dense(xt, np.zeros(len(xt))), make_param(svm_type=0, kernel_type=2, gamma=0.004, C=4.0),
           monkeypatch)


@pytest.mark.parametrize("kt,extra", [(0, {}), (1, dict(gamma=0.1, degree=3, coef0=0.5)), (3, dict(gamma=0.05, coef0=0.1))])
@pytest.mark.parametrize("d", [12, 150])
def test_other_kernels(kt, extra, d, monkeypatch):
    rng = np.random.default_rng(700 + kt + d)
    x, y = _blobs(rng, 3, 70, d)
    xt, _ = _blobs(np.random.default_rng(800 + kt + d), 3, 17, d)
    if d > 100:
        x, xt = x * 0.2, xt * 0.2
    _check(D.from_dense(x, y), D.from_dense(xt, np.zeros(len(xt))), make_param(svm_type=0, kernel_type=kt, C=1.0, **extra),
           monkeypatch)


@pytest.mark.parametrize("svm_type,extra", [(3, dict(p=0.1, C=5.0)), (4, dict(nu=0.4, C=5.0)), (2, dict(nu=0.2)), (1, dict(nu=0.3))])
def test_other_models(svm_type, extra, monkeypatch):
    rng = np.random.default_rng(900 + svm_type)
    x = rng.standard_normal((500, 9)).astype(np.float32)
    y = np.sin(x[:, 0]) + 0.3 * x[:, 1] if svm_type in (3, 4) else np.where(x[:, 0] + x[:, 1] > 0, 1.0, -1.0)
    xt = rng.standard_normal((130, 9)).astype(np.float32)
    _check(D.from_dense(x, y), D.from_dense(xt, np.zeros(len(xt))), make_param(svm_type=svm_type, kernel_type=2, gamma=0.2, **extra),
           monkeypatch)


@pytest.mark.parametrize("batch", [1, 63, 64, 65, 1000, -1])
def test_batch_sizes(batch, monkeypatch):
    rng = np.random.default_rng(77)
    x, y = _blobs(rng, 4, 300, 20)
    xt, _ = _blobs(np.random.default_rng(78), 4, 50, 20)
    _check(D.from_dense(x, y), D.from_dense(xt, np.zeros(len(xt))), make_param(svm_type=0, kernel_type=2, gamma=0.1, C=2.0),
           monkeypatch, batch=batch)


def test_test_rows_with_other_feature_ranges(monkeypatch):
    """Features the support vectors do not have are dropped from the products but stay in the row's self dot product
    (kernelmatrix.cpp:290-295,392); rows with fewer features than the support vectors are padded."""
    rng = np.random.default_rng(5)
    x, y = _blobs(rng, 3, 100, 10)
    tr = D.from_dense(x, y)
    wide = np.concatenate([_blobs(np.random.default_rng(6), 3, 20, 10)[0], rng.standard_normal((60, 7)).astype(np.float32)], axis=1)
    narrow = _blobs(np.random.default_rng(7), 3, 20, 10)[0][:, :4]
    for xt in (wide, narrow):
        _check(tr, D.from_dense(xt, np.zeros(len(xt))), make_param(svm_type=0, kernel_type=2, gamma=0.3, C=4.0), monkeypatch)


def test_long_chunks_and_many_support_vectors(monkeypatch):
    """Enough support vectors and rows that workgroups walk chunks of many column tiles."""
    rng = np.random.default_rng(11)
    x = rng.standard_normal((20000, 16)).astype(np.float32)
    y = np.where(np.sin(3 * x[:, 0]) * x[:, 1] + 0.3 * rng.standard_normal(20000) > 0, 1.0, -1.0)
    xt = rng.standard_normal((9000, 16)).astype(np.float32)
    gm, _ = _check(D.from_dense(x, y), D.from_dense(xt, np.zeros(len(xt))), make_param(svm_type=0, kernel_type=2, gamma=0.5, C=1.0),
                   monkeypatch)
    assert gm.total_sv > 8000


def test_sparse_class_pair_whose_rows_are_all_empty():
    """A wide, sparse three-class problem in which two classes' rows hold no feature at all: their class pair is a CSR
    sub-problem without a single stored entry (every kernel value is kappa(0, 0)), so there is nothing to slice for the
    CSR kernels; training and prediction still agree with the oracle."""
    rng = np.random.default_rng(3)
    ptr, col, val, y = [0], [], [], []
    for i in range(12):
        cls = i % 3 + 1
        if cls == 3:
            c = np.sort(rng.choice(np.arange(1, 400), 3, replace=False))
            col += list(c)
            val += list(rng.standard_normal(3).astype(np.float32))
        ptr.append(len(col))
        y.append(float(cls))
    tr = D.CsrData(ptr, col, val, y)
    xt = rng.standard_normal((4, 399)).astype(np.float32) * (rng.random((4, 399)) < 0.01)
    te = D.from_dense(xt, np.zeros(4))
    prm = make_param(svm_type=0, kernel_type=2, gamma=0.01, C=1.0)
    gm = Model(0).train(tr, prm)
    om = O.Model(tr.ptr, tr.col, tr.val, tr.y, _oparam(prm))
    assert gm.total_sv == om.total_sv and np.array_equal(gm.coef, om.coef) and np.array_equal(gm.rho, om.rho)
    _, gdec = gm.predict(te)
    _, odec = om.predict(te.ptr, te.col, te.val, 100)
    assert np.abs(gdec - odec).max() < 1e-6
