"""Pins the oracle's probability functions (sigmoidTrain, sigmoidPredict, multiclass_probability; reference
svc.cpp:197-430) against what the mathematics fixes: the reference holds no golden values for them.

* sigmoid_train minimises the regularised negative log likelihood of Platt's model: compared with a general-purpose
  minimiser of the same function, and the gradient at the result is below the routine's own 1e-5 stop.
* sigmoid_predict is 1 / (1 + exp(A*dec + B)).
* multiclass_probability solves min sum_{i<j} (r_ji p_i - r_ij p_j)^2 subject to sum p = 1: for two classes the
  answer is (r_01, r_10); for more the result is compared with the solution of the problem's KKT linear system.
"""
import numpy as np
import pytest
from scipy import optimize

import oracle_lib as O


def _nll(ab, dec, t):
    v = dec * ab[0] + ab[1]
    return np.sum(np.where(v >= 0, t * v + np.log1p(np.exp(-np.abs(v))), (t - 1) * v + np.log1p(np.exp(-np.abs(v)))))


@pytest.mark.parametrize("seed,n,shift", [(0, 200, 0.0), (1, 57, 0.8), (2, 1000, -0.3)])
def test_sigmoid_train_minimises_platts_likelihood(seed, n, shift):
    rng = np.random.default_rng(seed)
    lab = np.where(rng.random(n) < 0.4, 1, -1).astype(np.int32)
    dec = lab * 1.2 + rng.standard_normal(n) + shift
    a, b = O.sigmoid_train(dec, lab)
    n1, n0 = (lab > 0).sum(), (lab <= 0).sum()
    t = np.where(lab > 0, (n1 + 1.0) / (n1 + 2.0), 1.0 / (n0 + 2.0))
    best = optimize.minimize(_nll, [0.0, np.log((n0 + 1.0) / (n1 + 1.0))], args=(dec, t), method="BFGS",
                             options=dict(gtol=1e-9))
    assert abs(a - best.x[0]) < 1e-4 and abs(b - best.x[1]) < 1e-4
    assert _nll([a, b], dec, t) <= best.fun + 1e-8
    p = 1.0 / (1.0 + np.exp(dec * a + b))
    assert abs(np.sum(dec * (t - p))) < 1e-5 and abs(np.sum(t - p)) < 1e-5      # the routine's stopping rule
    assert a < 0                                                                 # larger decision value, larger P(+1)


def test_sigmoid_predict_closed_form():
    for dec, a, b in [(0.3, -1.7, 0.2), (-4.0, -2.0, 0.5), (50.0, -3.0, 0.0), (-50.0, -3.0, 0.0), (0.0, 0.0, 0.0)]:
        want = 1.0 / (1.0 + np.exp(dec * a + b))
        assert abs(O.sigmoid_predict(dec, a, b) - want) <= 1e-15 * max(1.0, want) + 1e-300


def _pairwise(rng, k):
    r = np.zeros((k, k))
    for i in range(k):
        for j in range(i + 1, k):
            r[i, j] = rng.uniform(0.05, 0.95)
            r[j, i] = 1 - r[i, j]
    return r


def test_multiclass_probability_two_classes():
    r = np.array([[0.0, 0.73], [0.27, 0.0]])
    p = O.multiclass_probability(r)
    assert np.abs(p - [0.73, 0.27]).max() < 5e-3     # the iteration stops at an error of 0.005 / k


@pytest.mark.parametrize("k,seed", [(3, 0), (4, 1), (7, 2), (12, 3)])
def test_multiclass_probability_solves_the_coupling_problem(k, seed):
    rng = np.random.default_rng(seed)
    r = _pairwise(rng, k)
    p = O.multiclass_probability(r)
    assert abs(p.sum() - 1) < 1e-9 and (p > 0).all()
    # Q of the quadratic form p'Qp = sum_{i<j} (r_ji p_i - r_ij p_j)^2, minimised subject to sum p = 1
    q = np.zeros((k, k))
    for i in range(k):
        for j in range(k):
            q[i, j] = np.sum(np.delete(r[:, i], i) ** 2) if i == j else -r[j, i] * r[i, j]
    kkt = np.block([[q, np.ones((k, 1))], [np.ones((1, k)), np.zeros((1, 1))]])
    want = np.linalg.solve(kkt, np.concatenate([np.zeros(k), [1.0]]))[:k]
    assert np.abs(p - want).max() < 0.005
    assert p @ q @ p <= want @ q @ want + 1e-4
    # consistent pairwise probabilities are recovered: r_ij = p_i / (p_i + p_j)
    truth = rng.dirichlet(np.ones(k) * 3)
    r2 = truth[:, None] / (truth[:, None] + truth[None, :])
    np.fill_diagonal(r2, 0)
    assert np.abs(O.multiclass_probability(r2) - truth).max() < 0.005
