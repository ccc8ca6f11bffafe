"""Pins for the oracle functions that no fixture of the reference covers, by what the mathematics fixes:

* NuSMOSolver::select_working_set (nusmosolver.cpp:48-118): an independent list restatement, brute force on
  small tie-heavy cases;
* NuSMOSolver::calculate_rho / scale_alpha_rho (nusmosolver.cpp:9-46,120-126): closed forms on hand-built f / alpha;
* the whole solver (selection + local solver + update_f + rho, all five SVM types): with an RBF kernel on distinct
  points the dual is strictly convex, so alpha*y and rho are unique; run to a KKT gap of 1e-8 the oracle must agree
  with LibSVM (scikit-learn) solving the same quadratic programme on the oracle's own kernel matrix.  A wrong sign,
  index, box bound, scaling or threshold anywhere in the chain moves the optimum far more than the 1e-6 allowed.
"""
import numpy as np
import pytest

import oracle_lib as O
from thundersvm_amd.data import from_dense


def is_up(a, y, C):
    return (y > 0 and a < C) or (y < 0 and a > 0)


def is_low(a, y, C):
    return (y > 0 and a > 0) or (y < 0 and a < C)


def _select_nu_brute(f, y, alpha, C, marked, k):
    """nusmosolver.cpp:48-118 with explicit candidate lists: per round one pick each from (I_up, y>0) and
    (I_up, y<0) in ascending (f, index) order, then (I_low, y>0) and (I_low, y<0) in descending order; an
    instance already taken (by any side or kept from the previous working set) is skipped; every pick but the
    first of a round is made only while fewer than k are selected."""
    n = len(f)
    order = sorted(range(n), key=lambda i: (f[i], i))
    sides = [
        [i for i in order if y[i] > 0 and is_up(alpha[i], y[i], C)],
        [i for i in order if y[i] < 0 and is_up(alpha[i], y[i], C)],
        [i for i in reversed(order) if y[i] > 0 and is_low(alpha[i], y[i], C)],
        [i for i in reversed(order) if y[i] < 0 and is_low(alpha[i], y[i], C)],
    ]
    taken = set(int(v) for v in marked)
    out = []
    while len(out) < k:
        progressed = False
        for s, cand in enumerate(sides):
            while cand and cand[0] in taken:
                cand.pop(0)
            if cand and (s == 0 or len(out) < k):
                out.append(cand[0])
                taken.add(cand.pop(0))
                progressed = True
        if not progressed:
            break
    return out


@pytest.mark.parametrize("seed", range(12))
def test_select_working_set_nu_brute_force(seed):
    rng = np.random.default_rng(100 + seed)
    n = int(rng.integers(12, 96))
    y = np.where(rng.random(n) < (0.5 if seed % 3 else 0.2), 1, -1).astype(np.int32)
    alpha = rng.choice([0.0, 0.3, 1.0], size=n, p=[0.4, 0.3, 0.3])
    f = np.round(rng.standard_normal(n), 1) if seed % 2 else -y.astype(float)   # heavy ties either way
    k = int(4 * rng.integers(1, max(2, n // 8)))
    marked = rng.permutation(n)[:k // 2].astype(np.int32) if seed % 4 else np.zeros(0, dtype=np.int32)
    want = _select_nu_brute(f, y, alpha, 1.0, marked, k)
    if len(want) < k:
        pytest.skip("fewer candidates than requested: the reference's loop would not terminate")
    got = O.select_working_set(f, y, alpha, 1.0, 1.0, marked, k, nu=True)
    assert list(got) == want[:k]
    assert len(set(got.tolist())) == k and not (set(got.tolist()) & set(marked.tolist()))


def test_select_working_set_nu_one_side_runs_dry():
    """A side without candidates is passed over; the others fill the set in the same rotation."""
    y = np.array([1, 1, 1, 1, -1, -1, -1, -1], dtype=np.int32)
    alpha = np.array([0, 0, 0, 0, 0, 0, 0, 0], dtype=float)   # y>0: I_up only; y<0: I_low only
    f = np.array([4, 3, 2, 1, 5, 6, 7, 8], dtype=float)
    got = O.select_working_set(f, y, alpha, 1.0, 1.0, np.zeros(0, dtype=np.int32), 6, nu=True)
    # rounds: (up,+) ascending f -> 3, 2, 1;  (low,-) descending f -> 7, 6, 5
    assert list(got) == [3, 7, 2, 6, 1, 5]


def _rho(f, y, alpha, C, nu, for_svr):
    import ctypes as Ct
    f = np.ascontiguousarray(f, dtype=np.float64)
    y = np.ascontiguousarray(y, dtype=np.int32)
    a = np.array(alpha, dtype=np.float64)
    rho = O.lib().orc_calculate_rho(O._ptr(f, Ct.c_double), O._ptr(y, Ct.c_int), O._ptr(a, Ct.c_double), Ct.c_int(len(f)),
                                    Ct.c_double(C), Ct.c_double(C), Ct.c_int(int(nu)), Ct.c_int(int(for_svr)))
    return rho, a


def test_calculate_rho_nu_closed_forms():
    C = 1.0
    y = np.array([1, 1, 1, -1, -1, -1], dtype=np.int32)
    # free vectors on both sides: r1 = mean f over free y>0, r2 = mean of -f over free y<0
    alpha = np.array([0.5, 0.25, 1.0, 0.5, 0.0, 0.75])
    f = np.array([0.2, 0.6, -3.0, -0.3, 9.0, -0.5])
    r1, r2 = (0.2 + 0.6) / 2, (0.3 + 0.5) / 2
    rho, a = _rho(f, y, alpha, C, True, True)
    assert rho == (r1 - r2) / 2 and np.array_equal(a, alpha)            # nu-SVR: no rescaling
    rho, a = _rho(f, y, alpha, C, True, False)
    r = (r1 + r2) / 2
    assert rho == ((r1 - r2) / 2) / r and np.array_equal(a, alpha / r)   # nu-SVC: alpha and rho divided by r
    # no free vector on the positive side: r1 = -(min over I_up of -f + max over I_low of -f) / 2
    alpha = np.array([0.0, 1.0, 1.0, 0.5, 0.0, 0.75])
    up_p = min(-f[0:1])                       # y>0, a<C: index 0
    low_p = max(-f[1:3])                      # y>0, a>0: indices 1, 2
    r1 = -(up_p + low_p) / 2
    rho, _ = _rho(f, y, alpha, C, True, True)
    assert rho == (r1 - r2) / 2
    # C-SMO for contrast: mean f over all free vectors (csmosolver.cpp:167-187)
    alpha = np.array([0.5, 0.25, 1.0, 0.5, 0.0, 0.75])
    rho, _ = _rho(f, y, alpha, C, False, False)
    assert rho == (0.2 + 0.6 - 0.3 - 0.5) / 4
    alpha = np.array([0.0, 1.0, 1.0, 1.0, 0.0, 0.0])                     # none free: -(up + low) / 2
    up = min(f[[0, 3]])
    low = max(f[[1, 2, 4, 5]])
    rho, _ = _rho(f, y, alpha, C, False, False)
    assert rho == -(up + low) / 2


def unique_optimum_problem():
    """Distinct points, RBF kernel (strictly convex dual), class +1 first so that grouped order = input order and
    the positive class of both solvers is the same."""
    rng = np.random.default_rng(3)
    n = 240
    y = np.where(np.arange(n) < n // 2, 1.0, -1.0)
    x = (rng.standard_normal((n, 5)) + 0.7 * y[:, None]).astype(np.float32)
    t = np.sin(x[:, 0]) + 0.5 * x[:, 1] ** 2 + 0.1 * rng.standard_normal(n)
    return x, y, t


def unique_optimum_cases():
    from sklearn.svm import SVC, NuSVC, SVR, NuSVR, OneClassSVM
    return [
        ("c_svc", O.C_SVC, dict(C=10.0), SVC(kernel="precomputed", C=10.0, tol=1e-10)),
        ("nu_svc", O.NU_SVC, dict(nu=0.3), NuSVC(kernel="precomputed", nu=0.3, tol=1e-10)),
        ("one_class", O.ONE_CLASS, dict(nu=0.2), OneClassSVM(kernel="precomputed", nu=0.2, tol=1e-10)),
        ("epsilon_svr", O.EPSILON_SVR, dict(C=10.0, p=0.1), SVR(kernel="precomputed", C=10.0, epsilon=0.1, tol=1e-10)),
        ("nu_svr", O.NU_SVR, dict(C=10.0, nu=0.4), NuSVR(kernel="precomputed", C=10.0, nu=0.4, tol=1e-10)),
    ]


def libsvm_optimum(sk, svm_type, K, target):
    """(alpha*y per instance, rho, decision values) of LibSVM's solution of the same problem."""
    sk.fit(K) if svm_type == O.ONE_CLASS else sk.fit(K, target)
    coef = np.zeros(len(K))
    coef[sk.support_] = sk.dual_coef_[0]
    rho = sk.offset_[0] if svm_type == O.ONE_CLASS else -sk.intercept_[0]
    dec = sk.decision_function(K) if svm_type in (O.C_SVC, O.NU_SVC, O.ONE_CLASS) else sk.predict(K)
    return coef, rho, dec


@pytest.mark.parametrize("case", range(5))
def test_unique_optimum_against_libsvm(case):
    x, y, t = unique_optimum_problem()
    name, st, prm, sk = unique_optimum_cases()[case]
    target = t if st in (O.EPSILON_SVR, O.NU_SVR) else y
    d = from_dense(x, target)
    p = O.make_param(st, O.RBF, gamma=0.5, epsilon=1e-8, C_=prm.get("C", 1.0), nu=prm.get("nu", 0.5), p=prm.get("p", 0.1))
    m = O.Model(d.ptr, d.col, d.val, d.y, p)
    K = O.KernelMatrix(d.ptr, d.col, d.val, p).get_rows(np.arange(d.n))
    coef, rho, dec = libsvm_optimum(sk, st, K, target)
    mine = np.zeros(d.n)
    mine[m.sv_indices] = m.coef
    _, odec = m.predict(d.ptr, d.col, d.val)
    assert np.abs(mine - coef).max() < 1e-6 * max(1.0, np.abs(coef).max()), name
    assert abs(m.rho[0] - rho) < 1e-6 * max(1.0, abs(rho)), name
    assert np.abs(odec[:, 0] - dec).max() < 1e-6, name


# ---------------------------------------------------------------------------------------------
# The reference's SyncMem counter at get_working_set_size (svmmodel.cpp:437-451), restated in the oracle
# ---------------------------------------------------------------------------------------------
def _reference_bytes_brute(x, held=0):
    """x: dense [m, nf] array whose non-zeros are the stored entries.  The column split of
    kernelmatrix.cpp:16-74 written with running sums over the sorted column counts."""
    m, nf = x.shape
    cnt = (x != 0).sum(axis=0)
    order = sorted(range(nf), key=lambda c: (cnt[c], c))
    sparse_cols = []
    total = 0
    for rank, c in enumerate(order, start=1):
        total += cnt[c]
        cells_taken = m * rank
        if total / cells_taken > 0.05 or cnt[c] / m > 0.5 or 4 * total > m * nf - cells_taken:
            break
        sparse_cols.append(c)
    nnz = int(cnt.sum())
    dense_cols = nf - len(sparse_cols)
    nnz_sparse = int(cnt[sparse_cols].sum()) if sparse_cols else 0
    b = 12 * nnz + 4 * (m + 1) + 16 * m            # val, col_ind, row_ptr, self_dot, diag
    if dense_cols > 0:
        b += 8 * m * dense_cols                    # dense part, m x dense_cols doubles
    if dense_cols < nf and nnz_sparse > 0:
        b += 12 * nnz_sparse + 4 * (m + 1)         # sparse part as CSR
    return b + 20 * m + held                       # y, alpha, f


def _oracle_reference_bytes(x, held=0):
    import ctypes as Ct
    d = from_dense(x[:, 1:])                        # column c of x = feature id c (column 0 is never used)
    L = O.lib()
    L.orc_reference_bytes.restype = Ct.c_longlong
    ptr, col, val = O.csr_arrays(d.ptr, d.col, d.val)
    return L.orc_reference_bytes(Ct.c_int(d.n), O._ptr(ptr, Ct.c_longlong), O._ptr(col, Ct.c_int), O._ptr(val, Ct.c_double),
                                 Ct.c_int(x.shape[1]), Ct.c_longlong(held))


def test_reference_memory_counter():
    rng = np.random.default_rng(8)
    m = 400
    # hand-computed: 3 full columns + the unused column 0 -> column 0 alone goes to the sparse part (0 entries), the
    # dense part is m x 3, no sparse CSR is built
    x = np.zeros((m, 4), dtype=np.float32)
    x[:, 1:] = 1 + rng.random((m, 3))
    want = 12 * 3 * m + 4 * (m + 1) + 16 * m + 8 * m * 3 + 20 * m
    assert _reference_bytes_brute(x) == want == _oracle_reference_bytes(x)
    # continuous columns plus one-hot groups (the 500k x 54 benchmark's shape): the rare indicator columns go sparse
    x = np.zeros((m, 55), dtype=np.float32)
    x[:, 1:11] = rng.standard_normal((m, 10))
    x[np.arange(m), 11 + rng.integers(0, 4, m)] = 1
    x[np.arange(m), 15 + rng.integers(0, 40, m)] = 1
    assert _reference_bytes_brute(x, 1000) == _oracle_reference_bytes(x, 1000)
    # text-like: everything sparse but a few head columns
    x = np.zeros((m, 300), dtype=np.float32)
    p = 1.0 / np.arange(1, 300) ** 1.1
    x[:, 1:] = (rng.random((m, 299)) < 6 * p) * rng.random((m, 299))
    assert _reference_bytes_brute(x) == _oracle_reference_bytes(x)
    # pixel-like, 20 % filled: no column qualifies for the sparse part except the unused one
    x = np.zeros((m, 65), dtype=np.float32)
    x[:, 1:] = (rng.random((m, 64)) < 0.2) * rng.random((m, 64))
    assert _reference_bytes_brute(x) == _oracle_reference_bytes(x)
