"""The C interface of the reference's Python package (include/thundersvm_scikit.h, reference
src/thundersvm/thundersvm-scikit.cpp), called the way python/thundersvm/thundersvm.py calls it: ctypes, float32
arrays, zero-based CSR columns.  Results are compared with the same training through the model-level ABI (which the
other GPU tests pin against the oracle) and with the reference's golden accuracy for its fixture."""
import ctypes as C
import os

import numpy as np
import pytest

import oracle_lib as O
from thundersvm_amd import data as D
from thundersvm_amd.model import Model, host_lib, make_param

pytestmark = pytest.mark.gpu
FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "test_dataset.txt")
_f, _i = C.POINTER(C.c_float), C.POINTER(C.c_int)


def _fp(a):
    return a.ctypes.data_as(_f)


def _ip(a):
    return a.ctypes.data_as(_i)


def _lib():
    lib = host_lib()
    lib.model_new.restype = C.c_void_p
    lib.save_to_string_scikit.restype = C.c_void_p
    return lib


def _fit(lib, data, svm_type, kernel, sparse, gamma=0.5, cost=10.0, nu=0.5, eps=0.1, tol=0.001, degree=3, coef0=0.0,
         probability=0, weights=None):
    """Mirrors SvmModel.fit of the reference's wrapper: returns (model handle, n_features, n_classes, succeed)."""
    m = lib.model_new(svm_type)
    y = np.ascontiguousarray(data.y, dtype=np.float32)
    wl = np.array(list((weights or {}).keys()), dtype=np.int32)
    wv = np.array(list((weights or {}).values()), dtype=np.float32)
    nf, nc, ok = (C.c_int * 1)(), (C.c_int * 1)(), (C.c_int * 1)()
    tail = (svm_type, kernel, degree, C.c_float(gamma), C.c_float(coef0), C.c_float(cost), C.c_float(nu), C.c_float(eps),
            C.c_float(tol), probability, len(wl), _ip(wl), _fp(wv), 0, -1, -1, -1, 0, nf, nc, ok, C.c_void_p(m))
    if sparse:
        val = np.ascontiguousarray(data.val, dtype=np.float32)
        ptr = np.ascontiguousarray(data.ptr, dtype=np.int32)
        col = np.ascontiguousarray(data.col - 1, dtype=np.int32)       # the wrapper passes scipy's zero-based indices
        lib.sparse_model_scikit(data.n, _fp(val), _ip(ptr), _ip(col), _fp(y), *tail)
    else:
        x = np.ascontiguousarray(data.to_dense(data.n_features + 1)[:, 1:], dtype=np.float32)
        lib.dense_model_scikit(data.n, x.shape[1], _fp(x), _fp(y), *tail)
    return m, nf[0], nc[0], ok[0]


def _predict(lib, m, data, sparse, n_binary):
    lab = np.zeros(data.n, dtype=np.float32)
    dec = np.zeros(data.n * n_binary, dtype=np.float32)
    if sparse:
        val = np.ascontiguousarray(data.val, dtype=np.float32)
        ptr = np.ascontiguousarray(data.ptr, dtype=np.int32)
        col = np.ascontiguousarray(data.col - 1, dtype=np.int32)
        assert lib.sparse_predict(data.n, _fp(val), _ip(ptr), _ip(col), C.c_void_p(m), _fp(lab), 0) == 0
        lib.sparse_decision(data.n, _fp(val), _ip(ptr), _ip(col), C.c_void_p(m), len(dec), _fp(dec))
    else:
        x = np.ascontiguousarray(data.to_dense(data.n_features + 1)[:, 1:], dtype=np.float32)
        assert lib.dense_predict(data.n, x.shape[1], _fp(x), C.c_void_p(m), _fp(lab), 0) == 0
        lib.dense_decision(data.n, x.shape[1], _fp(x), C.c_void_p(m), len(dec), _fp(dec))
    return lab, dec.reshape(data.n, n_binary)


@pytest.mark.parametrize("sparse", [True, False])
def test_csvc_fixture_through_the_scikit_interface(sparse):
    lib = _lib()
    d = D.load_libsvm(FIXTURE)
    m, n_features, n_classes, ok = _fit(lib, d, 0, 2, sparse, gamma=0.5, cost=100.0)
    assert ok == 1 and n_classes == 3 and n_features == d.n_features
    ref = Model(0).train(d, make_param(svm_type=0, kernel_type=2, gamma=0.5, C=100.0, epsilon=float(np.float32(0.001))))
    nb = (C.c_int * 1)()
    lib.get_n_binary_models(C.c_void_p(m), nb)
    assert nb[0] == 3 == ref.n_binary
    n_sv = lib.n_sv(C.c_void_p(m))
    assert n_sv == ref.total_sv
    # model parts, as the wrapper fetches them after fit
    row = np.zeros(n_sv + 1, dtype=np.int32)
    col = np.zeros(n_sv * n_features, dtype=np.int32)
    val = np.zeros(n_sv * n_features, dtype=np.float32)
    size, ind = (C.c_int * 1)(), np.zeros(n_sv, dtype=np.int32)
    lib.get_sv(_ip(row), _ip(col), _fp(val), size, _ip(ind), C.c_void_p(m))
    assert np.array_equal(ind, ref.sv_indices) and row[-1] == size[0]
    if sparse:
        assert np.array_equal(row, ref.sv_ptr) and np.array_equal(col[:size[0]], ref.sv_col)
        assert np.array_equal(val[:size[0]], ref.sv_val.astype(np.float32))
    coef = np.zeros((n_classes - 1) * n_sv, dtype=np.float32)
    lib.get_coef(_fp(coef), n_classes, n_sv, C.c_void_p(m))
    assert np.array_equal(coef, ref.coef.astype(np.float32))
    rho = np.zeros(3, dtype=np.float32)
    lib.get_rho(_fp(rho), 3, C.c_void_p(m))
    assert np.array_equal(rho, ref.rho.astype(np.float32))
    sup = np.zeros(3, dtype=np.int32)
    lib.get_support_classes(_ip(sup), 3, C.c_void_p(m))
    assert np.array_equal(sup, ref.n_sv)
    # prediction: labels, decision values, and the reference's golden accuracy (test_svc.cpp:33-37)
    lab, dec = _predict(lib, m, d, sparse, 3)
    rlab, rdec = ref.predict(d)
    assert np.array_equal(lab, rlab.astype(np.float32))
    assert np.array_equal(dec, rdec.astype(np.float32))
    assert abs((lab == d.y).mean() - 0.98) < 1e-5
    # model text round trip through the string functions
    sp = lib.save_to_string_scikit(C.c_void_p(m))
    text = C.string_at(sp)
    lib.free_string(C.c_void_p(sp))
    m2 = lib.model_new(0)
    lib.load_from_string_scikit(C.c_void_p(m2), text)
    kernel, deg, gam, c0, prob = C.create_string_buffer(20), (C.c_int * 1)(), (C.c_float * 1)(), (C.c_float * 1)(), (C.c_int * 1)()
    lib.init_model_param(kernel, deg, gam, c0, prob, C.c_void_p(m2))
    assert kernel.value == b"rbf" and gam[0] == 0.5 and deg[0] == 3 and prob[0] == 0
    nfeat = (C.c_int * 1)()
    lib.get_sv_max_index(C.c_void_p(m2), nfeat)
    assert nfeat[0] == d.n_features
    lab2, dec2 = _predict(lib, m2, d, sparse, 3)
    assert np.array_equal(lab2, lab) and np.abs(dec2 - dec).max() < 1e-5
    lib.model_free(C.c_void_p(m))
    lib.model_free(C.c_void_p(m2))


def test_regression_linear_coefficients_and_class_weights():
    lib = _lib()
    d = D.load_libsvm(FIXTURE)
    # epsilon-SVR through the sparse entry point (test_svr.cpp:35-39 parameters)
    m, _, _, ok = _fit(lib, d, 3, 2, True, gamma=0.25, cost=10.0, eps=0.1)
    assert ok == 1
    # (the interface carries tube width and tolerance as floats)
    ref = Model(3).train(d, make_param(svm_type=3, kernel_type=2, gamma=0.25, C=10.0, p=float(np.float32(0.1)),
                                       epsilon=float(np.float32(0.001))))
    val, dec = _predict(lib, m, d, True, 1)
    rval, _ = ref.predict(d)
    assert np.array_equal(val, rval.astype(np.float32))
    lib.model_free(C.c_void_p(m))
    # linear kernel: w = sum of coef * sv per binary model reproduces the decision values
    m, n_features, n_classes, ok = _fit(lib, d, 0, 0, False, cost=10.0)
    assert ok == 1
    w = np.zeros(3 * n_features, dtype=np.float32)
    lib.get_linear_coef(_fp(w), 3, n_features, C.c_void_p(m))
    rho = np.zeros(3, dtype=np.float32)
    lib.get_rho(_fp(rho), 3, C.c_void_p(m))
    lab, dec = _predict(lib, m, d, False, 3)
    x = d.to_dense(d.n_features + 1)[:, 1:]
    assert np.abs(x @ w.reshape(3, n_features).T - rho - dec).max() < 1e-3
    lib.model_free(C.c_void_p(m))
    # class weights reach the solver: the weighted class gets a larger box
    m, _, _, ok = _fit(lib, d, 0, 2, True, gamma=0.5, cost=1.0, weights={int(d.y[0]): 5.0})
    assert ok == 1
    ref = Model(0).train(d, make_param(svm_type=0, kernel_type=2, gamma=0.5, C=1.0, epsilon=float(np.float32(0.001)),
                                       weights={int(d.y[0]): 5.0}))
    n_sv = lib.n_sv(C.c_void_p(m))
    coef = np.zeros(2 * n_sv, dtype=np.float32)
    lib.get_coef(_fp(coef), 3, n_sv, C.c_void_p(m))
    assert np.array_equal(coef, ref.coef.astype(np.float32)) and np.abs(coef).max() > 1.0
    lib.model_free(C.c_void_p(m))


def test_failures_are_reported_through_succeed():
    lib = _lib()
    d = D.load_libsvm(FIXTURE)
    m, _, _, ok = _fit(lib, d, 1, 2, True, gamma=0.5, nu=0.999)    # nu infeasible for the smallest class pair
    assert ok == -1
    lib.model_free(C.c_void_p(m))
    m, _, _, ok = _fit(lib, d, 0, 7, True, gamma=0.5)    # no such kernel: the kernel-level ABI refuses it
    assert ok == -1
    lib.model_free(C.c_void_p(m))


def test_probability_estimates_with_class_weights():
    """The five fold models of a probability run train with the class weights of the run (svc.cpp:428-462 hands them
    the same parameters): probabilities against the oracle's, which differ visibly from the unweighted ones."""
    lib = _lib()
    d = D.load_libsvm(FIXTURE)
    weights = {int(d.y[0]): 6.0, int(d.y[-1]): 0.25}
    m, _, n_classes, ok = _fit(lib, d, 0, 2, True, gamma=0.5, cost=0.5, probability=1, weights=weights)
    assert ok == 1 and n_classes == 3
    lab, dec = _predict(lib, m, d, True, 3)
    prob = np.zeros(d.n * 3, dtype=np.float32)
    lib.get_pro(C.c_void_p(m), _fp(prob))
    prob = prob.reshape(d.n, 3)
    want = {}
    for name, w in (("weighted", weights), ("plain", None)):
        op = O.make_param(svm_type=0, kernel_type=2, gamma=0.5, C_=0.5, epsilon=float(np.float32(0.001)), expf_mode=1, weights=w)
        pa, pb = O.probability_train(d.ptr, d.col, d.val, d.y, op)
        om = O.Model(d.ptr, d.col, d.val, d.y, op)
        want[name] = O.predict_probability(om.predict_dec_values(d.ptr, d.col, d.val), pa, pb, 3)
    assert np.abs(prob - want["weighted"]).max() < 1e-6
    assert np.abs(want["weighted"] - want["plain"]).max() > 1e-3      # the weights matter on this problem
    lib.model_free(C.c_void_p(m))


@pytest.mark.parametrize("sparse", [True, False])
def test_probability_estimates(sparse):
    """probability = 1 (svc.cpp:137-143, 289-314, 432-491): probA / probB from the 5-fold decision values, coupled
    class probabilities per predicted row (get_pro), labels by highest probability; against the oracle, whose
    probability functions tests/test_oracle_probability.py pins."""
    lib = _lib()
    d = D.load_libsvm(FIXTURE)
    m, _, n_classes, ok = _fit(lib, d, 0, 2, sparse, gamma=0.5, cost=100.0, probability=1)
    assert ok == 1 and n_classes == 3
    lab, dec = _predict(lib, m, d, sparse, 3)
    prob = np.zeros(d.n * 3, dtype=np.float32)
    lib.get_pro(C.c_void_p(m), _fp(prob))
    prob = prob.reshape(d.n, 3)
    op = O.make_param(svm_type=0, kernel_type=2, gamma=0.5, C_=100.0, epsilon=float(np.float32(0.001)), expf_mode=1)
    pa, pb = O.probability_train(d.ptr, d.col, d.val, d.y, op)
    om = O.Model(d.ptr, d.col, d.val, d.y, op)
    want = O.predict_probability(om.predict_dec_values(d.ptr, d.col, d.val), pa, pb, 3)
    assert np.abs(prob - want).max() < 1e-6
    assert np.abs(prob.sum(axis=1) - 1).max() < 1e-6
    assert np.array_equal(lab, om.label[np.argmax(want, axis=1)].astype(np.float32))
    assert (lab == d.y).mean() > 0.95
    # probA / probB travel in the model text
    sp = lib.save_to_string_scikit(C.c_void_p(m))
    text = C.string_at(sp)
    lib.free_string(C.c_void_p(sp))
    assert b"probA" in text and b"probB" in text
    got_a = np.array(text.split(b"probA ")[1].split(b"\n")[0].split(), dtype=np.float64)
    got_b = np.array(text.split(b"probB ")[1].split(b"\n")[0].split(), dtype=np.float64)
    np.testing.assert_allclose(got_a, pa, rtol=1e-5)
    np.testing.assert_allclose(got_b, pb, rtol=1e-5, atol=1e-7)
    m2 = lib.model_new(0)
    lib.load_from_string_scikit(C.c_void_p(m2), text)
    kernel, deg, gam, c0, pr = C.create_string_buffer(20), (C.c_int * 1)(), (C.c_float * 1)(), (C.c_float * 1)(), (C.c_int * 1)()
    lib.init_model_param(kernel, deg, gam, c0, pr, C.c_void_p(m2))
    assert pr[0] == 1
    lab2, _ = _predict(lib, m2, d, sparse, 3)
    prob2 = np.zeros(d.n * 3, dtype=np.float32)
    lib.get_pro(C.c_void_p(m2), _fp(prob2))
    assert np.array_equal(lab2, lab) and np.abs(prob2.reshape(d.n, 3) - prob).max() < 1e-4   # six digits in the text
    lib.model_free(C.c_void_p(m))
    lib.model_free(C.c_void_p(m2))
