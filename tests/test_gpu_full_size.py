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


def _check_binary_problem(a, f, ysub, Cp, Cn, eps, rho):
    """Dual constraints, the stopping rule on the returned f and rho of one C-SVC sub-problem (alpha*y and f in the
    sub-problem's own order)."""
    alpha = a * ysub
    cmax = np.where(ysub > 0, Cp, Cn)
    assert alpha.min() >= 0 and np.all(alpha <= cmax)
    assert abs(a.sum()) < 1e-9 * max(Cp, Cn) * max(1.0, np.count_nonzero(a) ** 0.5)
    up = ((ysub > 0) & (alpha < cmax)) | ((ysub < 0) & (alpha > 0))
    low = ((ysub > 0) & (alpha > 0)) | ((ysub < 0) & (alpha < cmax))
    assert f[low].max() - f[up].min() < eps
    free = (alpha > 0) & (alpha < cmax)
    if free.any():
        assert abs(rho - f[free].mean()) < 1e-9
    else:
        assert abs(rho + (f[up].min() + f[low].max()) / 2) < 1e-9
    return alpha, free


@pytest.mark.parametrize("kernel", ["rbf", "linear"])
def test_c3_full_size_sparse_csvc(kernel):
    """72,000 x 20,958 CSR rows through the sparse get_rows kernel, both kernels of the benchmark configuration."""
    w = D.workload_c3(kernel=kernel)
    tr, p = w["train"], w["params"]
    prm = make_param(**p)
    eps, C_ = prm.epsilon, p["C"]
    gm = Model(0).train(tr, prm, keep_binary=True)
    a, f = gm.binary(0)
    n = tr.n
    lab0, lab1 = gm.label
    perm = np.concatenate([np.flatnonzero(tr.y == lab0), np.flatnonzero(tr.y == lab1)])
    ysub = np.concatenate([np.ones((tr.y == lab0).sum()), -np.ones((tr.y == lab1).sum())])
    alpha, free = _check_binary_problem(a, f, ysub, C_, C_, eps, gm.rho[0])
    assert free.any() and gm.total_sv == int((alpha > 0).sum())
    # f from scratch on a sample of instances, by the oracle's kernel rows
    rng = np.random.default_rng(7)
    pick = rng.choice(n, 48, replace=False)
    km = O.KernelMatrix(tr.ptr, tr.col, tr.val, _oparam(prm))
    a_orig = np.zeros(n)
    a_orig[perm] = a
    f_ref = km.get_rows(perm[pick]) @ a_orig - ysub[pick]
    np.testing.assert_allclose(f[pick], f_ref, rtol=0, atol=1e-8)
    # Karush-Kuhn-Tucker conditions of every training instance, from the model's own predictions
    lab, dec = gm.predict(tr)
    margin = ysub * dec[perm, 0]
    tol = eps + 1e-6
    assert np.all(margin[alpha == 0] >= 1 - tol)
    assert np.all(np.abs(margin[free] - 1) <= tol)
    assert np.all(margin[alpha == C_] <= 1 + tol)
    # decision values of sampled rows against the oracle's kernel sum over the model's support vectors
    ts = tr.rows(rng.choice(n, 96, replace=False))
    lab_t, dec_t = gm.predict(ts)
    ref = _oracle_decision(gm, prm, ts)
    assert np.abs(dec_t[:, 0] - ref).max() < 1e-6
    assert np.array_equal(lab_t, np.where(ref > 0, lab0, lab1))


def test_c4_full_size_seven_class_csvc():
    """500,000 x 54, 21 class pairs solved two at a time with slices of the row arena: the six largest pairs run with a
    partial row cache, the others with every row stored."""
    w = D.workload_c4(n_test=4000)
    tr, te, p = w["train"], w["test"], w["params"]
    prm = make_param(**p)
    eps, C_ = prm.epsilon, p["C"]
    gm = Model(0).train(tr, prm, keep_binary=True)
    k = len(gm.label)
    assert k == 7 and gm.n_binary == 21
    groups = [np.flatnonzero(tr.y == c) for c in gm.label]      # grouped order: classes by first appearance
    rng = np.random.default_rng(8)
    is_sv = np.zeros(tr.n, dtype=bool)
    b = 0
    partial = 0
    for i in range(k):
        for j in range(i + 1, k):
            a, f = gm.binary(b)
            ids = np.concatenate([groups[i], groups[j]])
            ysub = np.concatenate([np.ones(len(groups[i])), -np.ones(len(groups[j]))])
            assert len(a) == len(ids)
            alpha, free = _check_binary_problem(a, f, ysub, C_, C_, eps, gm.rho[b])
            is_sv[ids[alpha > 0]] = True
            st = gm.stats(b)
            assert st["ws_size"] == 1024 and st["n_iter"] >= 1
            partial += 0 < st["cache_rows"] < len(ids)
            # f from scratch on a few instances of the pair, by the oracle's kernel rows over the pair's rows
            sub = tr.rows(ids)
            km = O.KernelMatrix(sub.ptr, sub.col, sub.val, _oparam(prm))
            pick = rng.choice(len(ids), 6, replace=False)
            f_ref = km.get_rows(pick) @ a - ysub[pick]
            np.testing.assert_allclose(f[pick], f_ref, rtol=0, atol=1e-8)
            b += 1
    assert partial >= 1                                          # the large pairs did run with a partial cache
    assert gm.total_sv == int(is_sv.sum())
    assert np.array_equal(gm.sv_indices, np.concatenate([g[is_sv[g]] for g in groups]))
    # decision values of test rows against the oracle's kernel sum, and the one-vs-one vote (svc.cpp:265-288)
    ts = te.rows(rng.choice(te.n, 128, replace=False))
    lab, dec = gm.predict(ts)
    km = O.KernelMatrix(gm.sv_ptr, gm.sv_col, gm.sv_val, _oparam(prm))
    kv = km.get_rows_instances(ts.ptr, ts.col, ts.val)
    start = np.concatenate([[0], np.cumsum(gm.n_sv)[:-1]]).astype(np.int32)
    ref = O.sum_kernel_values(gm.coef.reshape(k - 1, gm.total_sv), gm.total_sv, start, gm.n_sv, gm.rho, kv, k, ts.n)
    assert np.abs(dec - ref).max() < 1e-6
    votes = np.zeros((ts.n, k), dtype=int)
    b = 0
    for i in range(k):
        for j in range(i + 1, k):
            votes[:, i] += ref[:, b] > 0
            votes[:, j] += ~(ref[:, b] > 0)
            b += 1
    clear = np.abs(ref).min(axis=1) > 1e-6                       # rows without a decision value on the margin
    assert np.array_equal(lab[clear], np.asarray(gm.label)[votes.argmax(axis=1)][clear])
    lab_all, _ = gm.predict(te)
    assert (lab_all == te.y).mean() > 0.8
