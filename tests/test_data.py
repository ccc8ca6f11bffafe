"""Host-side data handling: LibSVM text round trip (float32 rounding on load) and the seeded workloads."""
import numpy as np

from thundersvm_amd import data as D


def test_libsvm_round_trip(tmp_path):
    w = D.workload_c4(scale=0.002)
    path = str(tmp_path / "c4.txt")
    D.save_libsvm(path, w["train"])
    back = D.load_libsvm(path)
    assert np.array_equal(back.ptr, w["train"].ptr) and np.array_equal(back.col, w["train"].col)
    assert np.array_equal(back.val, w["train"].val) and np.array_equal(back.y, w["train"].y)


def test_values_are_float32_exact_and_seeded():
    for gen in (D.workload_c1, D.workload_c2, D.workload_c3, D.workload_c4, D.workload_c5):
        a, b = gen(0.01), gen(0.01)
        v = a["train"].val
        assert np.array_equal(v, v.astype(np.float32).astype(np.float64))
        assert np.array_equal(v, b["train"].val) and np.array_equal(a["train"].y, b["train"].y)


def test_workload_shapes():
    c4 = D.workload_c4(0.01)["train"]
    assert c4.n_features == 54 and set(np.unique(c4.y)) <= set(range(1, 8))
    assert np.all(np.diff(c4.ptr) == 12)                     # 10 continuous + 2 active one-hot columns
    c3 = D.workload_c3(0.01)["train"]
    assert c3.n_features <= 20958
    norms = np.sqrt(np.add.reduceat(c3.val ** 2, c3.ptr[:-1]))
    assert np.abs(norms - 1).max() < 1e-6
    c5 = D.workload_c5(0.01)
    assert c5["train"].n_features == 90 and np.all(np.diff(c5["train"].ptr) == 90)
    dense = c5["train"].to_dense()
    assert dense.shape[1] == 91 and np.all(dense[:, 0] == 0)
