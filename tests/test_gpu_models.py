"""GPU parity of whole training / prediction runs (host C++ layer + kernels) against the CPU oracle.

Modelled on the reference's model tests (src/test/test_svc.cpp, test_svr.cpp, test_nusvc.cpp,
test_nusvr.cpp, test_oneclass_svc.cpp: same fixture, same parameters, same golden values), then the
five benchmark workloads at reduced row counts.  Tolerances as stated for the path: coefficients
and rho 1e-6 relative, decision values 1e-6 absolute, labels identical; in practice the
trajectories are identical and the values agree to the last bit.
"""
import os

import numpy as np
import pytest

import oracle_lib as O
from thundersvm_amd import capi
from thundersvm_amd import data as D
from thundersvm_amd.data import load_libsvm
from thundersvm_amd.model import Dataset, Model, make_param

pytestmark = pytest.mark.gpu
FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "test_dataset.txt")


def _oparam(prm):
    return O.make_param(svm_type=prm.svm_type, kernel_type=prm.kernel_type, degree=prm.degree, gamma=prm.gamma,
                        coef0=prm.coef0, C_=prm.C, nu=prm.nu, p=prm.p, epsilon=prm.epsilon, max_iter=prm.max_iter,
                        max_mem_size=prm.max_mem_size, expf_mode=1)


def _compare(train, test, prm, ws=0, trace=8):
    gm = Model(prm.svm_type).train(train, prm, ws_override=ws, keep_binary=True, trace_cap=trace)
    om = O.Model(train.ptr, train.col, train.val, train.y, _oparam(prm), ws_override=ws, want_trace=True)
    gd, gw = gm.trace()
    od, ow = om.trace()
    k = min(len(gd), len(od), trace)
    if k:
        assert np.array_equal(gw[:k], ow[:k]), "working sets diverge at outer iteration %d" % np.flatnonzero(
            (gw[:k] != ow[:k]).any(axis=1))[0]
        assert np.array_equal(gd[:k], od[:k])
    for b in range(gm.n_binary):
        st = gm.stats(b)
        assert st["n_iter"] == om.n_iter[b] and st["local_iter"] == om.local_iter[b]
        ga, gf = gm.binary(b)
        oa, of = om.binary(b)
        np.testing.assert_allclose(ga, oa, rtol=1e-6, atol=1e-12)
        np.testing.assert_allclose(gf, of, rtol=1e-6, atol=1e-9)
    assert gm.total_sv == om.total_sv
    assert np.array_equal(gm.n_sv, om.n_sv) and np.array_equal(gm.sv_indices, om.sv_indices)
    np.testing.assert_allclose(gm.rho, om.rho, rtol=1e-6, atol=1e-12)
    np.testing.assert_allclose(gm.coef, om.coef, rtol=1e-6, atol=1e-12)
    tst = test if test is not None else train
    glab, gdec = gm.predict(tst, 100)
    olab, odec = om.predict(tst.ptr, tst.col, tst.val, 100)
    # (an infeasible nu leaves rho = 0/0 in the reference, nusmosolver.cpp:9-46, and decision values without a number)
    assert np.array_equal(np.isnan(gdec), np.isnan(odec))
    # 1e-6 as stated for the path, plus what the order of summation can move when the coefficients are huge and
    # cancel (nu-SVC divides alpha by a margin r that can be nearly zero, nusmosolver.cpp:120-126): the reference sums
    # one support vector after the other, the device kernel in a tree
    finite = np.isfinite(gm.coef)
    sd = np.add.reduceat(np.append(tst.val * tst.val, 0.0), np.minimum(tst.ptr[:-1], len(tst.val))) * (np.diff(tst.ptr) > 0)
    sd_max = max(float(sd.max(initial=0.0)), float((train.val * train.val).sum() / max(train.n, 1)) * 4, 1.0)
    k_max = {0: sd_max, 1: abs(prm.gamma * sd_max + prm.coef0) ** prm.degree, 2: 1.0, 3: 1.0}[prm.kernel_type]
    tol = 1e-6 + 1e-12 * float(np.abs(gm.coef[finite]).sum()) * max(k_max, 1.0)
    assert gdec.size == 0 or np.isnan(gdec).all() or np.nanmax(np.abs(gdec - odec)) < tol
    if tol < 1e-4:
        clear = np.nanmin(np.abs(odec), axis=1) > tol if odec.size else np.zeros(0, dtype=bool)   # (a value within tol of zero may fall on either side)
        assert np.array_equal(glab[clear], olab[clear]) or prm.svm_type in (3, 4)
        if prm.svm_type in (3, 4):
            assert np.abs(glab - olab).max() < 1e-6
    return gm, om, glab, tst


def test_fixture_csvc():            # test_svc.cpp:33-37
    d = D.load_libsvm(FIXTURE)
    gm, om, lab, tst = _compare(d, d, make_param(svm_type=0, kernel_type=2, gamma=0.5, C=100))
    assert abs((lab == d.y).mean() - 0.98) < 1e-5


def test_fixture_svr():             # test_svr.cpp:35-39
    d = D.load_libsvm(FIXTURE)
    gm, om, lab, tst = _compare(d, d, make_param(svm_type=3, kernel_type=2, gamma=0.5, C=100))
    assert abs(((lab - d.y) ** 2).mean() - 0.020752) < 1e-3


def test_fixture_nusvc():           # test_nusvc.cpp:40-44
    d = D.load_libsvm(FIXTURE)
    gm, om, lab, tst = _compare(d, d, make_param(svm_type=1, kernel_type=2, gamma=0.5, nu=0.1, C=100))
    assert abs((lab == d.y).mean() - 0.98) < 1e-3


def test_fixture_nusvr():           # test_nusvr.cpp:38-42
    d = D.load_libsvm(FIXTURE)
    gm, om, lab, tst = _compare(d, d, make_param(svm_type=4, kernel_type=2, gamma=0.5, nu=0.1, C=100))
    assert abs(((lab - d.y) ** 2).mean() - 0.028369) < 1.2e-5


def test_fixture_oneclass(tmp_path):   # test_oneclass_svc.cpp:7-30: train, save, load, predict
    d = D.load_libsvm(FIXTURE)
    gm, om, lab, tst = _compare(d, d, make_param(svm_type=2, kernel_type=2, gamma=0.5, nu=0.1))
    path = str(tmp_path / "one_class.model")
    gm.save(path)
    m2 = Model(2).load(path)
    lab2, _ = m2.predict(d, 100)
    assert int((lab2 > 0).sum()) == 135


@pytest.mark.parametrize("kt,prm", [(0, {}), (1, dict(gamma=0.5, degree=3, coef0=0.1)), (3, dict(gamma=0.5, coef0=0.1))])
def test_fixture_other_kernels(kt, prm):
    d = D.load_libsvm(FIXTURE)
    _compare(d, d, make_param(svm_type=0, kernel_type=kt, C=10, **prm))


def test_workload_c1():
    w = D.workload_c1()
    _compare(w["train"], w["test"], make_param(**w["params"]), trace=64)


def test_workload_c2_small():
    w = D.workload_c2(scale=0.03)
    _compare(w["train"], w["test"], make_param(**w["params"]), trace=64)


@pytest.mark.parametrize("kernel", ["linear", "rbf"])
def test_workload_c3_small(kernel):
    w = D.workload_c3(scale=0.04, kernel=kernel)
    _compare(w["train"], None, make_param(**w["params"]), trace=64)


def test_workload_c4_small():
    w = D.workload_c4(scale=0.01, n_test=500)
    _compare(w["train"], w["test"], make_param(**w["params"]), trace=64)


@pytest.mark.parametrize("kernel", ["linear", "rbf"])
def test_sparse_multiclass(kernel):
    """Four classes on sparse text-like rows (CSR layout on the device): the class pairs run side by side, each on the
    CSR kernels, and every pair's trajectory, alpha, f, rho and the assembled coefficients equal the oracle's."""
    w = D.workload_c3(scale=0.05, kernel=kernel)
    tr = w["train"]
    rng = np.random.default_rng(3)
    proj = rng.standard_normal((4, tr.n_features + 1))
    scores = np.zeros((tr.n, 4))
    for r in range(tr.n):
        cols = tr.col[tr.ptr[r]:tr.ptr[r + 1]]
        scores[r] = proj[:, cols] @ tr.val[tr.ptr[r]:tr.ptr[r + 1]]
    y = scores.argmax(axis=1).astype(np.float64) + 1.0
    y[rng.random(tr.n) < 0.05] = 4.0          # skewed class sizes and some label noise
    from thundersvm_amd.data import CsrData
    tr4 = CsrData(tr.ptr, tr.col, tr.val, y)
    gm, om, _, _ = _compare(tr4, None, make_param(**w["params"]), trace=16)
    assert gm.n_binary == 6


def test_workload_c5_small():
    w = D.workload_c5(scale=0.01)
    _compare(w["train"], w["test"], make_param(**w["params"]), trace=64)


@pytest.mark.parametrize("wl,scale", [("c1", 1.0), ("c2", 0.03), ("c3", 0.04), ("c4", 0.01), ("c5", 0.004)])
def test_untraced_training_matches_the_oracle(wl, scale):
    """Without a trace the production schedule runs: the next selection is enqueued ahead of the host's look at the
    stopping rule, update_f makes that selection's first pass, class pairs run side by side.  Same iteration counts,
    alpha, f, rho, coefficients and decision values as the oracle."""
    w = getattr(D, "workload_" + wl)(scale) if wl != "c1" else D.workload_c1()
    _compare(w["train"], w["test"], make_param(**w["params"]), trace=0)


def _csr(rows, y):
    ptr, col, val = [0], [], []
    for r in rows:
        for c, v in r:
            col.append(c)
            val.append(v)
        ptr.append(len(col))
    return D.CsrData(np.array(ptr, dtype=np.int64), np.array(col, dtype=np.int32),
                     np.array(val, dtype=np.float32).astype(np.float64), np.array(y, dtype=np.float64))


@pytest.mark.parametrize("case", ["two_points", "empty_rows", "duplicates_with_opposite_labels", "class_of_one",
                                  "exactly_one_working_set", "one_more_than_a_working_set", "feature_zero_only"])
@pytest.mark.parametrize("trace", [8, 0])
def test_degenerate_inputs(case, trace):
    """Inputs at the edges of what the reference accepts (dataset.cpp:190-234 groups whatever labels appear;
    kernelmatrix.cpp:183-205 takes rows without any feature): the smallest two-class problem, instances with no
    features, identical instances with opposite labels (alpha runs into C), a class with a single instance in a
    three-class problem, exactly one working set of instances and one more, and a data set whose only feature is
    feature 0.  All against the oracle, traced and with the production schedule."""
    rng = np.random.default_rng(17)
    prm = make_param(svm_type=0, kernel_type=2, gamma=0.5, C=10)
    if case == "two_points":
        d = _csr([[(1, 1.0)], [(1, -1.0), (2, 0.5)]], [1, -1])
    elif case == "empty_rows":
        rows = [[(c, float(v)) for c, v in zip(range(1, 6), rng.standard_normal(5))] for _ in range(60)]
        for i in (0, 7, 8, 59):
            rows[i] = []
        d = _csr(rows, np.where(np.arange(60) % 3 == 0, 1, -1))
    elif case == "duplicates_with_opposite_labels":
        base = [[(c, float(v)) for c, v in zip(range(1, 4), rng.standard_normal(3))] for _ in range(20)]
        d = _csr(base + base, [1] * 20 + [-1] * 20)
    elif case == "class_of_one":
        rows = [[(c, float(v)) for c, v in zip(range(1, 5), rng.standard_normal(4) + (i % 2))] for i in range(41)]
        d = _csr(rows, [i % 2 for i in range(40)] + [7])
    elif case in ("exactly_one_working_set", "one_more_than_a_working_set"):
        n = 1024 if case == "exactly_one_working_set" else 1025
        yy = np.where(rng.random(n) < 0.5, 1, -1)
        rows = [[(c, float(v)) for c, v in zip(range(1, 9), rng.standard_normal(8) + 0.3 * yy[i])] for i in range(n)]
        d = _csr(rows, yy)
    else:
        d = _csr([[(0, float(v))] for v in rng.standard_normal(50)], np.where(np.arange(50) % 2 == 0, 1, -1))
    _compare(d, d, prm, trace=trace)


def test_forced_working_set_larger_than_the_problem_is_rejected():
    """The working-set size can be forced for tests; one that the problem cannot fill is an error, not a selection
    that hands out instance ids of -1."""
    d = D.load_libsvm(FIXTURE)
    tiny = D.CsrData(d.ptr[:41], d.col[:d.ptr[40]], d.val[:d.ptr[40]], np.where(np.arange(40) % 2 == 0, 1.0, -1.0))
    with pytest.raises(RuntimeError, match="working-set size"):
        Model(0).train(tiny, make_param(svm_type=0, kernel_type=2, gamma=0.5, C=10), ws_override=64)
    Model(0).train(tiny, make_param(svm_type=0, kernel_type=2, gamma=0.5, C=10), ws_override=32)


def test_training_calls_from_two_threads_take_turns():
    """The row arena and the pooled streams are shared by all calls of a process: calls made from several host threads
    (ctypes releases the interpreter lock) are serialised by the library and give the models of sequential calls."""
    import threading
    w1, w2 = D.workload_c4(scale=0.004), D.workload_c5(scale=0.003)
    jobs = [(w1["train"], make_param(**w1["params"])), (w2["train"], make_param(**w2["params"]))]
    want = [Model(p.svm_type).train(d, p) for d, p in jobs]
    got = [None, None]

    def run(k):
        d, p = jobs[k]
        got[k] = Model(p.svm_type).train(d, p)

    for _ in range(3):
        threads = [threading.Thread(target=run, args=(k,)) for k in range(2)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        for k in range(2):
            assert got[k] is not None
            assert np.array_equal(got[k].coef, want[k].coef) and np.array_equal(got[k].rho, want[k].rho)
            assert np.array_equal(got[k].sv_indices, want[k].sv_indices)


def test_max_iter_cap():
    w = D.workload_c1(scale=0.5)
    prm = make_param(**w["params"])
    prm.max_iter = 3
    gm, om, _, _ = _compare(w["train"], w["test"], prm)
    assert gm.stats(0)["n_iter"] == 4


def test_row_cache_is_value_transparent():
    """The HBM kernel-row cache only changes which rows get recomputed: with it, without it and with a
    cache too small to keep everything the trained models are bit-identical."""
    w = D.workload_c2(scale=0.04)
    tr = w["train"]
    ref = None
    for cache_bytes in (0, -1, 1500 * tr.n * 8):
        prm = make_param(cache_bytes=cache_bytes, **w["params"])
        gm = Model(0).train(tr, prm, ws_override=256, keep_binary=True)
        st = gm.stats(0)
        if cache_bytes == 0:
            assert st["cache_rows"] == 0
        elif cache_bytes == -1:
            assert st["cache_rows"] == tr.n and st["cache_hits"] > 0
        else:
            assert 0 < st["cache_rows"] < tr.n
        a, f = gm.binary(0)
        cur = (a, f, gm.rho.copy(), st["n_iter"], st["local_iter"])
        if ref is None:
            ref = cur
        else:
            assert np.array_equal(cur[0], ref[0]) and np.array_equal(cur[1], ref[1])
            assert np.array_equal(cur[2], ref[2]) and cur[3:] == ref[3:]


def test_dataset_handle_and_file_loader(tmp_path):
    """Training from a DataSet handle, from CSR arrays and from a LibSVM text file gives the same model."""
    w = D.workload_c4(scale=0.004)
    tr = w["train"]
    prm = make_param(**w["params"])
    a = Model(0).train(tr, prm)
    b = Model(0).train(Dataset(tr), prm)
    path = str(tmp_path / "c4.txt")
    D.save_libsvm(path, tr)
    c = Model(0).train(Dataset(path=path), prm)
    ds = Dataset(tr).to_device()          # rows uploaded once; both trainings below take them from HBM
    d = Model(0).train(ds, prm)
    e = Model(0).train(ds, prm)
    for m in (b, c, d, e):
        assert np.array_equal(a.coef, m.coef) and np.array_equal(a.rho, m.rho) and np.array_equal(a.sv_indices, m.sv_indices)
    la, da = a.predict(tr)
    lb, db = b.predict(Dataset(tr))
    assert np.array_equal(da, db) and np.array_equal(la, lb)


def test_class_pairs_in_lockstep_give_the_same_model():
    """The pairs of a one-vs-one run are advanced one at a time or several in lockstep: identical models."""
    w = D.workload_c4(scale=0.01)
    tr = w["train"]
    ref = None
    for lanes, cache in ((1, -1), (2, -1), (3, 0), (5, 64 << 20), (8, -1), (0, -1)):
        m = Model(0).train(tr, make_param(pair_lanes=lanes, cache_bytes=cache, **w["params"]))
        cur = (m.coef.copy(), m.rho.copy(), m.sv_indices.copy(), [m.stats(b)["n_iter"] for b in range(m.n_binary)],
               [m.stats(b)["local_iter"] for b in range(m.n_binary)])
        xcds = [m.stats(b)["solver_xcd"] for b in range(m.n_binary)]
        if lanes != 1 and max(xcds) >= 0:   # (-1 everywhere: the lockstep schedule, no CU masks on this device)
            # every lane's local solver was elected onto an XCD of its own
            n_lanes = 8 if lanes == 0 else lanes
            assert all(0 <= x < n_lanes for x in xcds) and len(set(xcds)) >= 2, xcds
        if ref is None:
            ref = cur
            assert m.n_binary == 21
        else:
            assert np.array_equal(cur[0], ref[0]) and np.array_equal(cur[1], ref[1]) and np.array_equal(cur[2], ref[2])
            assert cur[3] == ref[3] and cur[4] == ref[4]


@pytest.mark.parametrize("wl", ["c1", "c5"])
def test_split_and_serial_schedules_give_the_same_model(wl, monkeypatch):
    """A task alone runs its local solver on compute units of its own, next to get_rows; with TSVM_NO_CU_SPLIT it
    runs every step in order on one stream.  Same trajectory, same model."""
    w = D.workload_c1(scale=0.5) if wl == "c1" else D.workload_c5(scale=0.005)
    tr, prm = w["train"], make_param(**w["params"])
    models = []
    for serial in (False, True):
        if serial:
            monkeypatch.setenv("TSVM_NO_CU_SPLIT", "1")
        m = Model(prm.svm_type).train(tr, prm, keep_binary=True)
        models.append((m.coef.copy(), m.rho.copy(), m.sv_indices.copy(), m.stats(0)["n_iter"], m.stats(0)["local_iter"],
                       m.binary(0)))
    a, b = models
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])
    assert a[3] == b[3] and a[4] == b[4]
    assert np.array_equal(a[5][0], b[5][0]) and np.array_equal(a[5][1], b[5][1])


@pytest.mark.parametrize("svm_type,extra,golden,metric", [
    (capi.C_SVC, dict(C=10.0), 0.973, "acc"),          # test_cross_validation.cpp:51-59
    (capi.NU_SVC, dict(), 0.660, "acc"),               # :61-68
    (capi.NU_SVR, dict(), 0.045, "mse"),               # :70-76
    (capi.EPSILON_SVR, dict(), 0.044, "mse"),          # :78-84
])
def test_cross_validation_goldens(svm_type, extra, golden, metric):
    """The reference's 5-fold cross-validation scores on its fixture (tolerance 1e-3, as in its tests)."""
    ds = Dataset(path=FIXTURE)
    y = load_libsvm(FIXTURE).y
    prm = make_param(svm_type=svm_type, kernel_type=capi.RBF, gamma=0.125, **extra)
    pred = Model(svm_type).cross_validation(ds, prm, 5)
    score = float(np.mean(pred == y)) if metric == "acc" else float(np.mean((pred - y) ** 2))
    assert abs(score - golden) < 1e-3, score


@pytest.mark.parametrize("case", range(5))
def test_unique_optimum_against_libsvm(case):
    """The GPU twin of tests/test_oracle_pins.py::test_unique_optimum_against_libsvm: with an RBF kernel on distinct
    points the dual has one optimum; trained to a KKT gap of 1e-8 the HIP path must reach LibSVM's solution of the
    same quadratic programme (kernel matrix taken from the GPU's own get_rows through the oracle's identical values):
    coefficients and rho 1e-6 relative, decision values 1e-6 absolute."""
    import test_oracle_pins as P
    x, y, t = P.unique_optimum_problem()
    name, st, prm, sk = P.unique_optimum_cases()[case]
    target = t if st in (O.EPSILON_SVR, O.NU_SVR) else y
    d = D.from_dense(x, target)
    gp = make_param(svm_type=st, kernel_type=capi.RBF, gamma=0.5, epsilon=1e-8, **prm)
    gm = Model(st).train(d, gp)
    K = O.KernelMatrix(d.ptr, d.col, d.val, _oparam(gp)).get_rows(np.arange(d.n))
    coef, rho, dec = P.libsvm_optimum(sk, st, K, target)
    mine = np.zeros(d.n)
    mine[gm.sv_indices] = gm.coef
    _, gdec = gm.predict(d)
    assert np.abs(mine - coef).max() < 1e-6 * max(1.0, np.abs(coef).max()), name
    assert abs(gm.rho[0] - rho) < 1e-6 * max(1.0, abs(rho)), name
    assert np.abs(gdec[:, 0] - dec).max() < 1e-6, name


def test_more_than_32_classes():
    """The reference's sum_kernel_values has no class limit (kernelmatrix_kernel.cpp:110-147): a 34-class model
    (561 class pairs) trains and predicts like the oracle's."""
    rng = np.random.default_rng(34)
    k, per, d = 34, 10, 6
    centres = 3.0 * rng.standard_normal((k, d))
    cls = rng.permutation(np.repeat(np.arange(k), per))
    x = (centres[cls] + 0.6 * rng.standard_normal((k * per, d))).astype(np.float32)
    tr = D.from_dense(x, (cls + 1).astype(np.float64))
    prm = make_param(svm_type=0, kernel_type=2, gamma=0.2, C=5.0)
    gm = Model(0).train(tr, prm)
    om = O.Model(tr.ptr, tr.col, tr.val, tr.y, _oparam(prm))
    assert gm.n_binary == 561 and gm.total_sv == om.total_sv
    np.testing.assert_allclose(gm.rho, om.rho, rtol=1e-6, atol=1e-12)
    np.testing.assert_allclose(gm.coef, om.coef, rtol=1e-6, atol=1e-12)
    glab, gdec = gm.predict(tr, 100)
    olab, odec = om.predict(tr.ptr, tr.col, tr.val, 100)
    assert np.abs(gdec - odec).max() < 1e-6 and np.array_equal(glab, olab)
    assert (glab == tr.y).mean() > 0.9


@pytest.mark.parametrize("svm_type,extra", [(3, dict(p=0.1)), (3, dict(p=0.0)), (4, dict(nu=0.4))])
def test_cache_switched_off_mid_run_on_a_stacked_problem(svm_type, extra, monkeypatch):
    """A row cache that has filled up and does not hit is switched off in mid-run (rotation between two slot
    tables from then on).  On the 2n-variable problems of SVR two working-set positions may share one stored row;
    after the switch every position must own a slot.  Same trajectory and model as without a cache, bit for bit.
    (The switch is made to happen at the first check, whatever the hit rate: TSVM_CACHE_OFF_BELOW is the percentage
    of a window's repeated lookups that must hit for the cache to stay.)"""
    monkeypatch.setenv("TSVM_CACHE_OFF_BELOW", "101")
    w = D.workload_c5(scale=0.01)
    tr = w["train"]
    p = dict(w["params"], svm_type=svm_type)
    p.update(extra)
    res = []
    for cache_bytes in (0, 5 << 20):
        m = Model(svm_type).train(tr, make_param(cache_bytes=cache_bytes, **p), ws_override=64, keep_binary=True)
        st = m.stats(0)
        assert st["cache_disabled"] == (cache_bytes != 0) and st["n_iter"] > 64
        res.append((m.coef.copy(), m.rho.copy(), m.sv_indices.copy(), st["n_iter"], st["local_iter"]) + m.binary(0))
    for a, b in zip(*res):
        assert np.array_equal(a, b)


def _ws_sizes(model, n_binary):
    return [model.stats(b)["ws_size"] for b in range(n_binary)]


@pytest.mark.parametrize("kind", ["mixed_3class", "svr", "csr_text"])
def test_working_set_size_follows_the_reference_memory_budget(kind):
    """SvmModel::get_working_set_size (svmmodel.cpp:437-451) subtracts what the reference's SyncMem counter holds from
    the -m budget.  With the budget set just around the point where floor(free / 8 / (n + n_features)) crosses 1024,
    the host layer's restated counter must flip the working-set size at the same byte as the oracle's."""
    rng = np.random.default_rng(77)
    if kind == "mixed_3class":
        w = D.workload_c4(scale=0.012)
        keep = np.flatnonzero(w["train"].y <= 3)
        tr, p = w["train"].rows(keep), dict(w["params"])
    elif kind == "svr":
        w = D.workload_c5(scale=0.006)
        tr, p = w["train"], dict(w["params"])
    else:
        w = D.workload_c3(scale=0.035)
        tr, p = w["train"], dict(w["params"])
    p["max_iter"] = 2                                   # the size is decided before the first iteration
    base = O.Model(tr.ptr, tr.col, tr.val, tr.y, _oparam(make_param(**p)))
    nb = base.n_binary
    L = O.lib()
    default = [L.orc_model_ws_size(base.h, b) for b in range(nb)]
    assert max(default) == 1024
    # bisect the budget at which the oracle's first problem drops from 1024 to 512
    lo, hi = 1 << 20, 8192 << 20
    while hi - lo > 1:
        mid = (lo + hi) // 2
        try:
            om = O.Model(tr.ptr, tr.col, tr.val, tr.y, _oparam(make_param(max_mem_size=mid, **p)))
            ok = L.orc_model_ws_size(om.h, 0) == 1024
        except Exception:
            ok = False
        lo, hi = (lo, mid) if ok else (mid, hi)
    flips = 0
    for budget in (hi - 4096, hi - 8, hi - 1, hi, hi + 1, hi + 4096, hi + (64 << 10), hi + (1 << 20)):
        prm = make_param(max_mem_size=budget, **p)
        om = O.Model(tr.ptr, tr.col, tr.val, tr.y, _oparam(prm))
        gm = Model(prm.svm_type).train(tr, prm)
        want = [L.orc_model_ws_size(om.h, b) for b in range(nb)]
        assert _ws_sizes(gm, nb) == want, (budget - hi, _ws_sizes(gm, nb), want)
        flips += want[0] == 1024
    assert 0 < flips < 8


def test_device_buffer_accounting_and_round_trip():
    """DeviceBuffer<T>, the device-only stand-in for SyncArray<T>: the checks of the reference's
    src/test/test_syncmem.cpp:7-50 and test_syncarray.cpp:7-60 that apply to a buffer without a host mirror
    (allocation counted once, released on destruction and on resize, moves transfer ownership without
    counting twice, upload -> download round trip), run by the test-only native library."""
    import selftest_lib
    lib = selftest_lib.lib()
    assert lib.tsvm_selftest_device_buffer() == 0, lib.tsvm_selftest_last_error()
