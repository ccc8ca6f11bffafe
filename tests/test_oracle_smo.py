"""Pins the oracle's SMO pieces with what the mathematics fixes: closed forms, invariants and brute
force on tiny inputs (the reference holds no fixture with alpha / rho / f values)."""
import itertools

import numpy as np
import pytest

import oracle_lib as O
from thundersvm_amd.data import from_dense


def is_up(a, y, Cp, Cn):
    return (y > 0 and a < Cp) or (y < 0 and a > 0)


def is_low(a, y, Cp, Cn):
    return (y > 0 and a > 0) or (y < 0 and a < Cn)


def test_predicates_and_max2power():
    L = O.lib()
    for a, y in itertools.product([0.0, 0.5, 1.0], [1.0, -1.0]):
        assert bool(L.orc_is_I_up(a, y, 1.0, 1.0)) == is_up(a, y, 1.0, 1.0)
        assert bool(L.orc_is_I_low(a, y, 1.0, 1.0)) == is_low(a, y, 1.0, 1.0)
        assert bool(L.orc_is_free(a, y, 1.0, 1.0)) == (0 < a < 1.0)
    assert [L.orc_max2power(v) for v in (1, 2, 3, 1023, 1024, 1025, 500000)] == [1, 2, 2, 512, 1024, 1024, 262144]
    # svmmodel.cpp:437-451 with the default 8192 MiB budget
    assert L.orc_working_set_size(3200, 33, 8192 << 20, 0) == 1024
    assert L.orc_working_set_size(150, 5, 8192 << 20, 0) == 128
    assert L.orc_working_set_size(800000, 91, 8192 << 20, 2 << 30) == 512
    assert L.orc_working_set_size(800000, 91, 8192 << 20, 1 << 30) == 1024


def test_sort_f_ties_by_index():
    f = np.array([1.0, -1.0, 1.0, -1.0, 0.0, -0.0, 1.0])
    assert list(O.sort_f(f)) == [1, 3, 4, 5, 0, 2, 6]


def _select_brute(f, y, alpha, C, marked, k):
    """csmosolver.cpp:123-165 restated with explicit lists."""
    order = sorted(range(len(f)), key=lambda i: (f[i], i))
    taken = set(marked)
    out, left, right = [], 0, len(f) - 1
    while len(out) < k:
        while left < len(f) and (order[left] in taken or not is_up(alpha[order[left]], y[order[left]], C, C)):
            left += 1
        if left < len(f):
            out.append(order[left]); taken.add(order[left])
        while right >= 0 and (order[right] in taken or not is_low(alpha[order[right]], y[order[right]], C, C)):
            right -= 1
        if right >= 0:
            out.append(order[right]); taken.add(order[right])
        if left >= len(f) and right < 0:
            break
    return out[:k] if len(out) >= k else out


@pytest.mark.parametrize("seed", range(6))
def test_select_working_set_brute_force(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(8, 64))
    y = np.where(rng.random(n) < 0.5, 1, -1).astype(np.int32)
    alpha = rng.choice([0.0, 0.3, 1.0], size=n)
    f = np.round(rng.standard_normal(n), 1) if seed % 2 else -y.astype(float)
    k = int(2 * rng.integers(1, n // 4 + 1))
    marked = rng.permutation(n)[:k // 2].astype(np.int32)
    got = O.select_working_set(f, y, alpha, 1.0, 1.0, marked, k)
    want = _select_brute(f, y, alpha, 1.0, marked, k)
    assert list(got[:len(want)]) == want
    sel = [g for g in got if g >= 0]
    assert len(set(sel)) == len(sel) and not (set(sel) & set(marked.tolist()))


def test_c_smo_two_point_closed_form():
    """One point per class: alpha_1 = alpha_2 = min(C, 2 / (K11 + K22 - 2 K12))."""
    for C, k12 in [(10.0, 0.3), (0.5, 0.3), (10.0, 0.9)]:
        K = np.array([[1.0, k12], [k12, 1.0]])
        y = np.array([1, -1], dtype=np.int32)
        a, ad, diff = O.c_smo_solve(y, -y.astype(float), np.zeros(2), [0, 1], C, C, K, np.ones(2), 2, 1e-9, 1000)
        want = min(C, 2.0 / (2.0 - 2.0 * k12))
        assert np.allclose(a, [want, want], rtol=1e-12)
        assert diff[0] == 2.0
        assert np.allclose(ad, [-want, want])


@pytest.mark.parametrize("nu", [False, True])
def test_local_solver_invariants(nu):
    rng = np.random.default_rng(5)
    n, ws, C = 400, 128, 2.0
    y = np.where(rng.random(n) < 0.5, 1, -1).astype(np.int32)
    x = (rng.standard_normal((n, 6)) + 0.5 * y[:, None]).astype(np.float32)
    d = from_dense(x)
    km = O.KernelMatrix(d.ptr, d.col, d.val, O.make_param(kernel_type=O.RBF, gamma=0.3))
    alpha = rng.choice([0.0, 0.7, C], size=n, p=[0.6, 0.3, 0.1])
    kfull = km.get_rows(np.arange(n))
    f = kfull @ (alpha * y) - y
    ids = rng.permutation(n)[:ws].astype(np.int32)
    k_rows = kfull[ids]
    fn = O.nu_smo_solve if nu else O.c_smo_solve
    args = (y, f, alpha, ids, C) if nu else (y, f, alpha, ids, C, C)
    a, ad, diff = fn(*args, k_rows, km.diag(), n, 1e-3, 100000)
    assert ((a >= 0) & (a <= C)).all()
    assert abs(((a - alpha) * y).sum()) < 1e-9                       # sum y alpha conserved
    assert np.array_equal(ad, -(a[ids] - alpha[ids]) * y[ids])
    assert np.array_equal(a[np.setdiff1d(np.arange(n), ids)], alpha[np.setdiff1d(np.arange(n), ids)])
    f_new = O.update_f(f, ad, k_rows, n)
    assert np.abs(f_new - (kfull @ (a * y) - y)).max() < 1e-9        # f stays the gradient
    if not nu:
        up = min(f_new[i] for i in ids if is_up(a[i], y[i], C, C))
        low = max(f_new[i] for i in ids if is_low(a[i], y[i], C, C))
        assert low - up < max(1e-3, np.float32(0.1) * diff[0]) + 1e-9   # local stopping rule
        assert diff[1] > 0


def test_update_f_skips_zeros_in_order():
    rng = np.random.default_rng(2)
    k = rng.random((6, 9))
    ad = np.array([0.5, 0.0, -1.25, 0.0, 0.0, 2.0])
    f = rng.random(9)
    want = f.copy()
    for j in range(9):
        s = 0.0
        for t in (0, 2, 5):
            s = float(np.float64(ad[t]) * k[t, j] + s)   # products are not exact here: compare to 1 ulp
        want[j] -= s
    assert np.abs(O.update_f(f, ad, k, 9) - want).max() < 1e-15


def test_full_solve_kkt_and_objective():
    rng = np.random.default_rng(9)
    n, C = 600, 5.0
    y = np.where(np.arange(n) % 2 == 0, 1, -1).astype(np.int32)
    x = (rng.standard_normal((n, 5)) + 0.8 * y[:, None]).astype(np.float32)
    d = from_dense(x)
    km = O.KernelMatrix(d.ptr, d.col, d.val, O.make_param(kernel_type=O.RBF, gamma=0.5))
    res = O.smo_solve(km, y, np.zeros(n), -y.astype(float), 1e-3, C, C, 512, trace_cap=64)
    a, f = res["alpha"], res["f"]
    kfull = km.get_rows(np.arange(n))
    assert np.abs(f - (kfull @ (a * y) - y)).max() < 1e-9
    assert abs((a * y).sum()) < 1e-9 and ((a >= 0) & (a <= C)).all()
    up = min(f[i] for i in range(n) if is_up(a[i], y[i], C, C))
    low = max(f[i] for i in range(n) if is_low(a[i], y[i], C, C))
    assert low - up < 1e-3 * 1.0001 + 1e-12          # global KKT gap below eps at exit
    free = (a > 0) & (a < C)
    assert abs(res["rho"] - f[free].mean()) < 1e-12
    obj = -(a.sum() - 0.5 * (a * y) @ kfull @ (a * y))
    assert abs(res["obj"] - obj) < 1e-6 * abs(obj)
    # working sets: no duplicates, first half = previous last half
    ws = res["trace_ws"]
    for it in range(len(ws)):
        assert len(set(ws[it].tolist())) == ws.shape[1]
        if it:
            assert np.array_equal(ws[it][:256], ws[it - 1][256:])
    # diff[0] of the trace ends below eps
    assert res["trace_diff"][-1][0] < 1e-3


def test_svr_identity():
    rng = np.random.default_rng(4)
    n = 300
    x = rng.standard_normal((n, 4)).astype(np.float32)
    t = np.sin(x[:, 0]) + 0.1 * rng.standard_normal(n)
    d = from_dense(x, t)
    p = O.make_param(O.EPSILON_SVR, O.RBF, gamma=0.5, C_=10.0, p=0.1)
    m = O.Model(d.ptr, d.col, d.val, d.y, p)
    a2, f2 = m.binary(0)          # alpha of the 2n-variable problem and its gradient
    km = O.KernelMatrix(d.ptr, d.col, d.val, p)
    k = km.get_rows(np.arange(n))
    beta = a2[:n] - a2[n:]
    assert np.abs(f2[:n] - (k @ beta + 0.1 - t)).max() < 1e-9      # f = K beta + p - y  (svr.cpp:24-29)
    assert np.abs(f2[n:] - (k @ beta - 0.1 - t)).max() < 1e-9
    pred, dec = m.predict(d.ptr, d.col, d.val)
    assert np.abs(dec[:, 0] - (k @ beta - m.rho[0])).max() < 1e-9
    assert ((pred - t) ** 2).mean() < 0.05


def test_sum_kernel_values_layout():
    """LibSVM coefficient layout (svmmodel.h:154-164, svc.cpp:86-108) by brute force."""
    rng = np.random.default_rng(1)
    cnt = np.array([3, 2, 4], dtype=np.int32)
    start = np.array([0, 3, 5], dtype=np.int32)
    T = 9
    coef = rng.standard_normal((2, T))
    rho = rng.standard_normal(3)
    k = rng.random((5, T))
    dec = O.sum_kernel_values(coef, T, start, cnt, rho, k, 3, 5)
    p = 0
    for i in range(3):
        for j in range(i + 1, 3):
            for r in range(5):
                s = sum(coef[j - 1, start[i] + l] * k[r, start[i] + l] for l in range(cnt[i]))
                s += sum(coef[i, start[j] + l] * k[r, start[j] + l] for l in range(cnt[j]))
                assert abs(dec[r, p] - (s - rho[p])) < 1e-12
            p += 1
