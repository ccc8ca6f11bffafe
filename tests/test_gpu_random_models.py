"""Random small problems through the whole training and prediction path, GPU against the CPU oracle: all five SVM
types, four kernels, one to 300 features at densities from 5 % to 100 % (so: instances without features, identical
instances, indicator columns), two to five classes of uneven size, forced and default working-set sizes, traced
(one pair at a time) and untraced (production schedule) runs, nu values that are infeasible for some class pairs.
The outer iterations are capped at 30: the comparison is of trajectories, not of converged models."""
import numpy as np
import pytest

from thundersvm_amd import data as D
from thundersvm_amd.model import make_param

import test_gpu_models as T

pytestmark = pytest.mark.gpu


def _case(seed):
    rng = np.random.default_rng(seed)
    svm_type = int(rng.choice([0, 0, 0, 1, 2, 3, 3, 4]))
    kt = int(rng.choice([0, 1, 2, 2, 2, 3]))
    n = int(rng.choice([3, 17, 64, 200, 700, 1500, 2600, 5000]))
    d = int(rng.choice([1, 2, 5, 20, 60, 130, 300]))
    dens = float(rng.choice([0.05, 0.3, 1.0]))
    n_cls = int(rng.choice([2, 2, 3, 5])) if svm_type in (0, 1) else 1
    x = rng.standard_normal((n, d)).astype(np.float32)
    x *= rng.random((n, d)) < dens
    if rng.random() < 0.3:   # the last columns as one group of indicator columns
        k = min(d, int(rng.integers(1, 6)))
        x[:, d - k:] = 0
        x[np.arange(n), d - k + rng.integers(0, k, size=n)] = 1.0
    if svm_type in (0, 1):
        w = rng.standard_normal(d)
        y = np.digitize(x @ w, np.quantile(x @ w, np.linspace(0, 1, n_cls + 1)[1:-1])).astype(np.float64)
        flip = rng.random(n) < 0.1
        y[flip] = rng.integers(0, n_cls, size=int(flip.sum()))
        if len(np.unique(y)) < 2:
            y[0], y[1] = 0, 1
        smallest = int(np.sort(np.bincount(y.astype(int))[np.bincount(y.astype(int)) > 0])[:2].sum())
    else:
        y = np.sin(x[:, 0]) + 0.1 * rng.standard_normal(n)
        smallest = n * (2 if svm_type in (3, 4) else 1)
    prm = dict(svm_type=svm_type, kernel_type=kt, C=float(rng.choice([0.1, 1, 10, 100])),
               gamma=float(rng.choice([0.01, 0.1, 0.5, 2])), coef0=float(rng.choice([0, 0.5])), degree=int(rng.choice([2, 3])),
               nu=float(rng.choice([0.1, 0.3, 0.5])), p=float(rng.choice([0.01, 0.1])))
    if kt == 1:
        prm["gamma"] = min(prm["gamma"], 0.1)
    if kt == 3:
        prm["gamma"] = min(prm["gamma"], 0.01)   # an indefinite kernel lets the reference's step leave [0, C] and overflow
    ws = int(rng.choice([0, 0, 64, 256]))
    if ws > smallest:
        ws = 0
    trace = int(rng.choice([0, 0, 16]))
    return D.from_dense(x, y), prm, ws, trace


@pytest.mark.parametrize("seed", range(7000, 7060))
def test_random_small_problem(seed):
    data, prm, ws, trace = _case(seed)
    T._compare(data, data, make_param(max_iter=30, **prm), ws=ws, trace=trace)


def _sparse_case(seed):
    """Few non-zeros among hundreds to thousands of features: the rows stay in CSR form on the device."""
    rng = np.random.default_rng(seed)
    svm_type = int(rng.choice([0, 0, 0, 1, 2, 3, 4]))
    kt = int(rng.choice([0, 1, 2, 2, 3]))
    n = int(rng.choice([5, 40, 300, 1100, 3000]))
    d = int(rng.choice([600, 3000, 21000]))
    avg = float(rng.choice([0.5, 3, 12]))
    n_cls = int(rng.choice([2, 2, 3, 4])) if svm_type in (0, 1) else 1
    cnt = rng.poisson(avg, size=n)
    ptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(cnt, out=ptr[1:])
    col = np.concatenate([np.sort(rng.choice(d, size=c, replace=False)) + 1 for c in cnt] + [np.zeros(0, dtype=np.int64)])
    val = rng.standard_normal(len(col)).astype(np.float32).astype(np.float64)
    if svm_type in (0, 1):
        y = rng.integers(0, n_cls, size=n).astype(np.float64)
        if len(np.unique(y)) < 2:
            y[0], y[1] = 0, 1
        smallest = int(np.sort(np.bincount(y.astype(int))[np.bincount(y.astype(int)) > 0])[:2].sum())
    else:
        y = rng.standard_normal(n)
        smallest = n * (2 if svm_type in (3, 4) else 1)
    prm = dict(svm_type=svm_type, kernel_type=kt, C=float(rng.choice([0.1, 1, 10])), gamma=float(rng.choice([0.01, 0.1, 0.5])),
               coef0=float(rng.choice([0, 0.5])), degree=int(rng.choice([2, 3])), nu=float(rng.choice([0.1, 0.3, 0.5])),
               p=float(rng.choice([0.01, 0.1])))
    if kt == 3:
        prm["gamma"] = 0.01
    ws = int(rng.choice([0, 0, 64, 256]))
    if ws > smallest:
        ws = 0
    trace = int(rng.choice([0, 0, 16]))
    return D.CsrData(ptr, col.astype(np.int32), val, y), prm, ws, trace


@pytest.mark.parametrize("seed", range(9000, 9040))
def test_random_sparse_problem(seed):
    data, prm, ws, trace = _sparse_case(seed)
    T._compare(data, data, make_param(max_iter=30, **prm), ws=ws, trace=trace)
