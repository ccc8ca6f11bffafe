"""The benchmark workloads at their full sizes, checked through properties that do not depend on the size.

The CPU oracle takes minutes to hours on these problems, so a run is not compared with an oracle run.
What is checked instead holds for every correct SMO solution and every correct kernel sum:
  * the box and equality constraints of the dual (svc.cpp:147-177, svr.cpp:29-62);
  * the stopping rule of the last outer iteration on the returned f (csmosolver.cpp:108-113): the largest
    f over I_low exceeds the smallest f over I_up by less than epsilon;
  * f, which the solver only ever updates incrementally (update_f, once per outer iteration), equals the
    kernel sum computed from scratch by the oracle's kernel rows, on a sample of instances;
  * the Karush-Kuhn-Tucker conditions of every training instance, from the model's own predictions;
  * decision values of a sample of test instances equal the oracle's kernel sum over the model's support
    vectors (1e-6 absolute, the tolerance of the path).
"""
import numpy as np
import pytest

import oracle_lib as O
from thundersvm_amd import data as D
from thundersvm_amd.model import Model, make_param

pytestmark = pytest.mark.gpu


def _oparam(prm):
    return O.make_param(svm_type=prm.svm_type, kernel_type=prm.kernel_type, degree=prm.degree, gamma=prm.gamma,
                        coef0=prm.coef0, C_=prm.C, nu=prm.nu, p=prm.p, epsilon=prm.epsilon, max_iter=prm.max_iter,
                        expf_mode=1)


def _oracle_decision(gm, prm, rows):
    """Kernel sum of the model's own support vectors and coefficients, by the oracle's kernel rows."""
    km = O.KernelMatrix(gm.sv_ptr, gm.sv_col, gm.sv_val, _oparam(prm))
    k = km.get_rows_instances(rows.ptr, rows.col, rows.val)          # [rows, n_sv]
    return k @ gm.coef - gm.rho[0]


def test_c2_full_size_binary_csvc():
    w = D.workload_c2()
    tr, te, p = w["train"], w["test"], w["params"]
    prm = make_param(**p)
    eps, C_ = prm.epsilon, p["C"]
    gm = Model(0).train(tr, prm, keep_binary=True)
    a, f = gm.binary(0)                                   # alpha*y and f, class-grouped order of the sub-problem
    n = tr.n
    lab0, lab1 = gm.label
    perm = np.concatenate([np.flatnonzero(tr.y == lab0), np.flatnonzero(tr.y == lab1)])
    ysub = np.concatenate([np.ones((tr.y == lab0).sum()), -np.ones((tr.y == lab1).sum())])
    assert len(a) == n and len(perm) == n
    alpha = a * ysub
    # dual constraints
    assert alpha.min() >= 0 and alpha.max() <= C_
    assert abs(a.sum()) < 1e-9 * C_
    # stopping rule on the returned f
    up = ((ysub > 0) & (alpha < C_)) | ((ysub < 0) & (alpha > 0))
    low = ((ysub > 0) & (alpha > 0)) | ((ysub < 0) & (alpha < C_))
    assert f[low].max() - f[up].min() < eps
    free = (alpha > 0) & (alpha < C_)
    assert free.any()
    assert abs(gm.rho[0] - f[free].mean()) < 1e-9
    # f from scratch on a sample of instances
    rng = np.random.default_rng(5)
    pick = rng.choice(n, 48, replace=False)
    km = O.KernelMatrix(tr.ptr, tr.col, tr.val, _oparam(prm))
    a_orig = np.zeros(n)
    a_orig[perm] = a
    f_ref = km.get_rows(perm[pick]) @ a_orig - ysub[pick]
    np.testing.assert_allclose(f[pick], f_ref, rtol=0, atol=1e-8)
    # support vectors are the instances with alpha > 0
    assert gm.total_sv == int((alpha > 0).sum())
    # Karush-Kuhn-Tucker conditions of all training instances, from the model's predictions
    _, dec = gm.predict(tr)
    margin = (ysub * dec[perm, 0])
    tol = eps + 1e-6
    assert np.all(margin[alpha == 0] >= 1 - tol)       # (with this gamma nearly every instance is a support vector)
    assert np.all(np.abs(margin[free] - 1) <= tol)
    assert np.all(margin[alpha == C_] <= 1 + tol)
    # decision values and labels of test instances against the oracle's kernel sum
    ts = te.rows(rng.choice(te.n, 128, replace=False))
    lab, dec_t = gm.predict(ts)
    ref = _oracle_decision(gm, prm, ts)
    assert np.abs(dec_t[:, 0] - ref).max() < 1e-6
    assert np.array_equal(lab, np.where(ref > 0, lab0, lab1))


def test_c5_full_size_epsilon_svr():
    w = D.workload_c5()
    tr, te, p = w["train"], w["test"], w["params"]
    prm = make_param(**p)
    eps, C_, tube = prm.epsilon, p["C"], p["p"]
    gm = Model(3).train(tr, prm)
    n = tr.n
    coef = gm.coef
    assert np.abs(coef).max() <= C_ and np.abs(coef).min() > 0
    assert abs(coef.sum()) < 1e-9 * C_ * gm.total_sv
    # the model's support vectors are the training rows its indices name
    sv = tr.rows(gm.sv_indices)
    assert np.array_equal(sv.ptr, gm.sv_ptr) and np.array_equal(sv.col, gm.sv_col) and np.array_equal(sv.val, gm.sv_val)
    # Karush-Kuhn-Tucker conditions of all training instances (svr.cpp:29-62 builds the 2n-variable problem
    # whose optimum they characterise), from the model's predictions
    c = np.zeros(n)
    c[gm.sv_indices] = coef
    val, _ = gm.predict(tr)
    r = tr.y - val
    tol = eps + 1e-6
    assert np.all(np.abs(r[c == 0]) <= tube + tol)
    assert np.all(np.abs(r[(c > 0) & (c < C_)] - tube) <= tol)
    assert np.all(np.abs(r[(c < 0) & (c > -C_)] + tube) <= tol)
    assert np.all(r[c == C_] >= tube - tol)
    assert np.all(r[c == -C_] <= -tube + tol)
    # predicted values of test instances against the oracle's kernel sum
    rng = np.random.default_rng(6)
    ts = te.rows(rng.choice(te.n, 64, replace=False))
    val_t, dec_t = gm.predict(ts)
    ref = _oracle_decision(gm, prm, ts)
    assert np.abs(dec_t[:, 0] - ref).max() < 1e-6
    assert np.abs(val_t - ref).max() < 1e-6
