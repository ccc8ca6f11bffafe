"""GPU parity: KernelMatrix::get_rows / diag and sum_kernel_values through the C ABI vs the CPU oracle.

Mirrors src/test/test_kernelmatrix.cpp (same fixture, same row sets, all four kernels) and adds
ragged shapes.  Bars: all four kernels bit-exact (the oracle runs its restated expf / powf / tanhf, expf_mode=1, which
tests/test_oracle_expf.py pins to libm; test_poly_and_sigmoid_rows_match_libm checks the GPU against libm itself);
decision values 1e-9.
"""
import numpy as np
import pytest
import torch

import gpu_util as G
import oracle_lib as O
from thundersvm_amd import capi
from thundersvm_amd.data import load_libsvm, from_dense, CsrData

pytestmark = pytest.mark.gpu
FIXTURE = __import__("os").path.join(__import__("os").path.dirname(__file__), "golden", "test_dataset.txt")

KERNELS = [
    ("rbf", O.RBF, dict(gamma=0.5)),
    ("poly", O.POLY, dict(gamma=0.5, degree=3, coef0=0.1)),
    ("linear", O.LINEAR, dict()),
    ("sigmoid", O.SIGMOID, dict(gamma=0.5, coef0=0.1)),
]


def _check(name, got, want):
    bad = np.flatnonzero(got.ravel() != want.ravel())
    assert bad.size == 0, "%s: %d mismatching entries, first %s got %r want %r" % (
        name, bad.size, bad[:1], got.ravel()[bad[:1]], want.ravel()[bad[:1]])


@pytest.mark.parametrize("name,kt,prm", [("poly3", O.POLY, dict(gamma=0.5, degree=3, coef0=0.1)),
                                         ("poly2", O.POLY, dict(gamma=1.5, degree=2, coef0=0.0)),
                                         ("poly5", O.POLY, dict(gamma=0.05, degree=5, coef0=1.0)),
                                         ("poly7neg", O.POLY, dict(gamma=-0.3, degree=7, coef0=-0.2)),
                                         ("poly0", O.POLY, dict(gamma=0.5, degree=0, coef0=0.1)),
                                         ("sigmoid", O.SIGMOID, dict(gamma=0.5, coef0=0.1)),
                                         ("sigmoid_small", O.SIGMOID, dict(gamma=1e-3, coef0=0.0)),
                                         ("sigmoid_large", O.SIGMOID, dict(gamma=9.0, coef0=-2.0))])
def test_poly_and_sigmoid_rows_match_libm(name, kt, prm):
    """The polynomial and sigmoid epilogues against the host's libm powf / tanhf themselves (the oracle with
    expf_mode=0 calls them, as the reference does, kernelmatrix_kernel.cpp:94-108): bit for bit, including negative
    arguments of odd powers, degree 0 and arguments on both sides of tanhf's ranges."""
    rng = np.random.default_rng(21)
    x = rng.standard_normal((300, 12)).astype(np.float32).astype(np.float64)
    x[::7] *= 40.0            # some large dot products: overflow and saturation
    x[3::11] *= 1e-3          # and some tiny ones
    data = from_dense(x, np.ones(300))
    okm = O.KernelMatrix(data.ptr, data.col, data.val, O.make_param(kernel_type=kt, expf_mode=0, **prm))
    x_d, nf, ld, sd, diag = _device_km(data, kt, prm)
    _check(name, G.host(diag), okm.diag())
    rows = np.arange(0, 300, 3, dtype=np.int32)
    got = G.get_rows_dense(x_d, ld, data.n, nf, sd, x_d, ld, G.dev(rows), len(rows), sd, kt, **prm)
    want = okm.get_rows(rows)
    both_nan = np.isnan(G.host(got)) & np.isnan(want)
    _check(name, np.where(both_nan, 0.0, G.host(got)), np.where(both_nan, 0.0, want))


def _device_km(data, kt, prm):
    xh, nf, ld = G.dense_padded(data)
    x_d = G.dev(xh)
    sd = torch.empty(data.n, dtype=torch.float64, device="cuda")
    capi.call("tsvm_dense_self_dot", G.ptr(x_d), ld, data.n, nf, G.ptr(sd), G.stream())
    diag = torch.empty(data.n, dtype=torch.float64, device="cuda")
    capi.call("tsvm_kernel_diag", G.ptr(sd), data.n, kt, prm.get("gamma", 0.0), prm.get("coef0", 0.0),
              prm.get("degree", 3), G.ptr(diag), G.stream())
    return x_d, nf, ld, sd, diag


@pytest.mark.parametrize("name,kt,prm", KERNELS)
def test_fixture_rows_and_diag(name, kt, prm):
    data = load_libsvm(FIXTURE)
    p = O.make_param(kernel_type=kt, expf_mode=1, **prm)
    okm = O.KernelMatrix(data.ptr, data.col, data.val, p)
    x_d, nf, ld, sd, diag = _device_km(data, kt, prm)
    assert nf == okm.n_features
    assert np.array_equal(G.host(sd), okm.self_dot())
    _check(name, G.host(diag), okm.diag())
    rows = np.arange(10, dtype=np.int32) * 3 + 4          # test_kernelmatrix.cpp:83-86
    rows_d = G.dev(rows)
    got = G.get_rows_dense(x_d, ld, data.n, nf, sd, x_d, ld, rows_d, len(rows), sd, kt, **prm)
    _check(name, G.host(got), okm.get_rows(rows))
    if kt != O.LINEAR:   # float rows are the same values in half the bytes
        got32 = G.get_rows_dense(x_d, ld, data.n, nf, sd, x_d, ld, rows_d, len(rows), sd, kt, row_type=capi.ROW_F32, **prm)
        assert np.array_equal(G.host(got32).astype(np.float64), G.host(got))
    # get_rows(instances): first 10 rows as an external batch (test_kernelmatrix.cpp:108-118)
    batch = data.rows(np.arange(10))
    bh = batch.to_dense(ld)
    b_d = G.dev(bh)
    sdb = torch.empty(10, dtype=torch.float64, device="cuda")
    capi.call("tsvm_dense_self_dot", G.ptr(b_d), ld, 10, ld, G.ptr(sdb), G.stream())
    got = G.get_rows_dense(x_d, ld, data.n, nf, sd, b_d, ld, None, 10, sdb, kt, **prm)
    _check(name, G.host(got), okm.get_rows_instances(batch.ptr, batch.col, batch.val))


@pytest.mark.parametrize("n,d,m,density", [(1, 1, 1, 1.0), (130, 9, 1, 1.0), (257, 33, 129, 1.0), (1000, 54, 512, 0.3),
                                           (515, 100, 64, 0.2), (2049, 784, 16, 0.2)])
@pytest.mark.parametrize("name,kt,prm", KERNELS[:1] + KERNELS[2:3])
def test_random_dense(name, kt, prm, n, d, m, density):
    rng = np.random.default_rng(n * 1000 + d)
    x = rng.standard_normal((n, d)).astype(np.float32)
    x[rng.random((n, d)) > density] = 0
    data = from_dense(x)
    if data.nnz == 0:
        data = from_dense(np.ones((n, d), dtype=np.float32))
    p = O.make_param(kernel_type=kt, expf_mode=1, **prm)
    okm = O.KernelMatrix(data.ptr, data.col, data.val, p)
    x_d, nf, ld, sd, diag = _device_km(data, kt, prm)
    idx = rng.integers(0, n, size=m).astype(np.int32)
    idx_d = G.dev(idx)
    got = G.get_rows_dense(x_d, ld, n, nf, sd, x_d, ld, idx_d, m, sd, kt, **prm)
    _check(name, G.host(got), okm.get_rows(idx))
    if kt != O.LINEAR:
        got32 = G.get_rows_dense(x_d, ld, n, nf, sd, x_d, ld, idx_d, m, sd, kt, row_type=capi.ROW_F32, **prm)
        assert got32.dtype == torch.float32 and np.array_equal(G.host(got32).astype(np.float64), G.host(got))


@pytest.mark.parametrize("seed", range(12))
def test_ragged_shapes_sweep(seed):
    """Seeded sweep over ragged shapes: feature counts around the 8/16-column K tiles, row and column counts around
    the 64/128-row tiles, with column subsets (x_idx), working-row subsets (a_idx) and scattered output slots at
    the same time; RBF, both row element types, bit for bit against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.choice([1, 2, 63, 64, 65, 127, 129, 255, 300, 641]))
    d = int(rng.choice([1, 3, 7, 8, 9, 15, 16, 17, 31, 33, 47, 48, 100, 129, 130, 257]))
    m = int(rng.choice([1, 31, 33, 64, 65, 127, 128, 130]))
    x = rng.standard_normal((n, d)).astype(np.float32)
    x[rng.random((n, d)) > 0.6] = 0
    x[:, -1] = rng.standard_normal(n).astype(np.float32)     # the last feature is used: n_features == d
    data = from_dense(x)
    kt, prm = O.RBF, dict(gamma=0.25)
    okm = O.KernelMatrix(data.ptr, data.col, data.val, O.make_param(kernel_type=kt, expf_mode=1, **prm))
    x_d, nf, ld, sd, _ = _device_km(data, kt, prm)
    cols = rng.permutation(n)[:max(1, n - int(rng.integers(0, 3)))].astype(np.int32)     # x_idx: a subset, permuted
    rows = rng.integers(0, n, size=m).astype(np.int32)
    slots = rng.permutation(m + 3)[:m].astype(np.int32)
    want = okm.get_rows(rows)[:, cols]
    cols_d, rows_d, slots_d = G.dev(cols), G.dev(rows), G.dev(slots)
    for row_type, dt in ((capi.ROW_F64, torch.float64), (capi.ROW_F32, torch.float32)):
        out = torch.full((m + 3, len(cols) + 5), -3.0, dtype=dt, device="cuda")
        capi.call("tsvm_get_rows_dense", G.ptr(x_d), ld, G.ptr(cols_d), len(cols), nf, G.ptr(sd), G.ptr(x_d), ld,
                  G.ptr(rows_d), m, G.ptr(sd), kt, prm["gamma"], 0.0, 3, G.ptr(out), row_type, G.ptr(slots_d),
                  len(cols) + 5, G.stream())
        got = G.host(out).astype(np.float64)
        assert np.array_equal(got[slots][:, :len(cols)], want), (n, d, m)
        assert (got[:, len(cols):] == -3.0).all()                 # nothing is written beyond the n columns
        untouched = np.setdiff1d(np.arange(m + 3), slots)
        assert (got[untouched] == -3.0).all()                     # nor into slots that were not named


def test_float_rows_rejected_for_linear_kernel():
    x_d = torch.zeros((8, 8), dtype=torch.float64, device="cuda")
    out = torch.zeros((8, 8), dtype=torch.float32, device="cuda")
    with pytest.raises(capi.TsvmError):
        capi.call("tsvm_get_rows_dense", G.ptr(x_d), 8, None, 8, 8, None, G.ptr(x_d), 8, None, 8, None, O.LINEAR, 0.0, 0.0, 3,
                  G.ptr(out), capi.ROW_F32, None, 8, G.stream())


def _sliced_copy(data, n, nf, val_type):
    """The stored rows in slices of 64 (tsvm_csr_slice_widths, tsvm_csr_to_sliced), checked against a numpy layout."""
    val_d, col_d, ptr_d = G.dev(data.val), G.dev(data.col), G.dev(data.ptr)
    n_slices = (n + 63) // 64
    widths = torch.zeros(n_slices, dtype=torch.int32, device="cuda")
    capi.call("tsvm_csr_slice_widths", G.ptr(ptr_d), n, G.ptr(widths), G.stream())
    lens = np.diff(data.ptr)
    want_w = np.array([lens[s * 64:(s + 1) * 64].max(initial=0) for s in range(n_slices)])
    assert np.array_equal(G.host(widths), want_w)
    sp = np.concatenate([[0], np.cumsum(64 * want_w)]).astype(np.int64)
    sp_d = G.dev(sp)
    ell_col = torch.full((int(sp[-1]),), -5, dtype=torch.int32, device="cuda")
    ell_val = torch.full((int(sp[-1]),), 7.0, dtype=torch.float32 if val_type == capi.ROW_F32 else torch.float64, device="cuda")
    capi.call("tsvm_csr_to_sliced", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), n, G.ptr(sp_d), nf, G.ptr(ell_col), G.ptr(ell_val),
              val_type, G.stream())
    ec, ev = G.host(ell_col), G.host(ell_val).astype(np.float64)
    for j in (0, 1, 63, 64, n // 2, n - 1):
        s, l = j // 64, j % 64
        ent = sp[s] + 64 * np.arange(want_w[s]) + l
        k = lens[j]
        assert np.array_equal(ec[ent[:k]], data.col[data.ptr[j]:data.ptr[j + 1]]) and (ec[ent[k:]] == nf).all()
        assert np.array_equal(ev[ent[:k]], data.val[data.ptr[j]:data.ptr[j + 1]]) and (ev[ent[k:]] == 0).all()
    return (val_d, col_d, ptr_d), sp_d, ell_col, ell_val


@pytest.mark.parametrize("n,d,m,max_k", [(700, 3000, 70, 40), (5000, 3000, 512, 40), (3000, 20958, 130, 90), (1000, 50, 16, 50),
                                         (333, 9000, 1, 30)])
@pytest.mark.parametrize("name,kt,prm", KERNELS)
def test_csr_sliced_path(name, kt, prm, n, d, m, max_k):
    """tsvm_get_rows_csr_sliced (stored rows streamed from their sliced copy, working rows as a tile in LDS) against the
    oracle's rows, bit for bit: skewed feature frequencies (a few features in almost every row, a long tail), empty rows,
    a working set that is not a multiple of sixteen, duplicates in the working set, output slots, both value types."""
    rng = np.random.default_rng(n + m)
    p_col = 1.0 / np.arange(1, d + 1) ** 1.1
    p_col /= p_col.sum()
    ptr, col, val = [0], [], []
    for i in range(n):
        k = int(rng.integers(0, max_k + 1)) if i % 7 else 0
        c = np.sort(rng.choice(d, size=min(k, d), replace=False, p=p_col)) + 1
        col.extend(c)
        val.extend(rng.standard_normal(len(c)).astype(np.float32))
        ptr.append(len(col))
    data = CsrData(ptr, col, np.asarray(val, dtype=np.float64))
    p = O.make_param(kernel_type=kt, expf_mode=1, **prm)
    okm = O.KernelMatrix(data.ptr, data.col, data.val, p)
    nf = okm.n_features
    max_nnz = int(np.diff(data.ptr).max())
    idx = rng.integers(0, n, size=m).astype(np.int32)
    if m > 3: idx[3] = idx[1]
    idx_d = G.dev(idx)
    want = okm.get_rows(idx)
    slots = rng.permutation(m + 5)[:m].astype(np.int32)
    slots_d = G.dev(slots)
    for val_type in (capi.ROW_F32, capi.ROW_F64):
        lds = capi.kernel_lib().tsvm_get_rows_csr_sliced_lds(nf, max_nnz, val_type)
        assert 0 < lds <= 160 * 1024, lds
        (val_d, col_d, ptr_d), sp_d, ell_col, ell_val = _sliced_copy(data, n, nf, val_type)
        sd = torch.empty(n, dtype=torch.float64, device="cuda")
        capi.call("tsvm_csr_self_dot", G.ptr(val_d), G.ptr(ptr_d), n, G.ptr(sd), G.stream())
        row_types = [capi.ROW_F64] if kt == O.LINEAR else [capi.ROW_F64, capi.ROW_F32]
        for rt in row_types:
            ldo = n + 3
            out = torch.full((m + 5, ldo), -3.0, dtype=torch.float32 if rt == capi.ROW_F32 else torch.float64, device="cuda")
            capi.call("tsvm_get_rows_csr_sliced", G.ptr(ell_col), G.ptr(ell_val), val_type, G.ptr(sp_d), n, G.ptr(sd), G.ptr(val_d),
                      G.ptr(col_d), G.ptr(ptr_d), G.ptr(idx_d), m, G.ptr(sd), nf, max_nnz, kt, prm.get("gamma", 0.0),
                      prm.get("coef0", 0.0), prm.get("degree", 3), G.ptr(out), rt, G.ptr(slots_d), ldo, G.stream())
            got = G.host(out).astype(np.float64)
            _check(name, got[slots][:, :n], want)
            untouched = np.setdiff1d(np.arange(m + 5), slots)
            assert (got[untouched] == -3.0).all() and (got[:, n:] == -3.0).all()
    # shapes the kernel does not take are refused: rows so long that eight of them overflow the tile, feature tables
    # larger than the LDS
    assert capi.kernel_lib().tsvm_get_rows_csr_sliced_lds(20000, 5000, capi.ROW_F32) == 0
    assert capi.kernel_lib().tsvm_get_rows_csr_sliced_lds(200000, 10, capi.ROW_F32) == 0


@pytest.mark.parametrize("n", [700, 5000])   # four / sixteen stored rows per workgroup
@pytest.mark.parametrize("name,kt,prm", KERNELS)
def test_csr_path(name, kt, prm, n):
    rng = np.random.default_rng(7)
    d, m = 3000, 70
    ptr = [0]
    col, val = [], []
    for i in range(n):
        k = rng.integers(0, 40)          # includes empty rows
        c = np.sort(rng.choice(d, size=k, replace=False)) + 1
        col.extend(c)
        val.extend(rng.standard_normal(k).astype(np.float32))
        ptr.append(len(col))
    data = CsrData(ptr, col, np.asarray(val, dtype=np.float64))
    p = O.make_param(kernel_type=kt, expf_mode=1, **prm)
    okm = O.KernelMatrix(data.ptr, data.col, data.val, p)
    nf = okm.n_features
    val_d, col_d, ptr_d = G.dev(data.val), G.dev(data.col), G.dev(data.ptr)
    sd = torch.empty(n, dtype=torch.float64, device="cuda")
    capi.call("tsvm_csr_self_dot", G.ptr(val_d), G.ptr(ptr_d), n, G.ptr(sd), G.stream())
    assert np.array_equal(G.host(sd), okm.self_dot())
    idx = rng.integers(0, n, size=m).astype(np.int32)
    idx_d = G.dev(idx)
    w = torch.empty((nf, m), dtype=torch.float64, device="cuda")
    capi.call("tsvm_csr_stage_rows", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), G.ptr(idx_d), m, nf, G.ptr(w), G.stream())
    sdw = torch.empty(m, dtype=torch.float64, device="cuda")
    capi.call("tsvm_gather_f64", G.ptr(sd), G.ptr(idx_d), m, G.ptr(sdw), G.stream())
    out = torch.empty((m, n), dtype=torch.float64, device="cuda")
    capi.call("tsvm_get_rows_csr", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), None, n, G.ptr(sd), G.ptr(w), m, G.ptr(sdw), kt,
              prm.get("gamma", 0.0), prm.get("coef0", 0.0), prm.get("degree", 3), G.ptr(out), capi.ROW_F64, None, n,
              G.stream())
    _check(name, G.host(out), okm.get_rows(idx))
    if kt != O.LINEAR:   # float rows hold the same values
        out32 = torch.empty((m, n), dtype=torch.float32, device="cuda")
        capi.call("tsvm_get_rows_csr", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), None, n, G.ptr(sd), G.ptr(w), m, G.ptr(sdw),
                  kt, prm.get("gamma", 0.0), prm.get("coef0", 0.0), prm.get("degree", 3), G.ptr(out32), capi.ROW_F32, None,
                  n, G.stream())
        assert np.array_equal(G.host(out32).astype(np.float64), G.host(out))
    # a staging matrix kept all-zero between uses, with float elements (the values are floats): rows scattered in,
    # the same bits out of the kernel, rows scattered out again
    for wt, dt in ((capi.ROW_F32, torch.float32), (capi.ROW_F64, torch.float64)):
        wz = torch.zeros((nf, m), dtype=dt, device="cuda")
        capi.call("tsvm_csr_scatter_rows", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), G.ptr(idx_d), m, nf, G.ptr(wz), wt, 0, G.stream())
        assert np.array_equal(G.host(wz).astype(np.float64), G.host(w))
        out_s = torch.empty((m, n), dtype=torch.float64, device="cuda")
        capi.call("tsvm_get_rows_csr_staged", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), None, n, G.ptr(sd), G.ptr(wz), wt, m,
                  G.ptr(sdw), kt, prm.get("gamma", 0.0), prm.get("coef0", 0.0), prm.get("degree", 3), G.ptr(out_s), capi.ROW_F64,
                  None, n, G.stream())
        assert np.array_equal(G.host(out_s), G.host(out))
        capi.call("tsvm_csr_scatter_rows", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), G.ptr(idx_d), m, nf, G.ptr(wz), wt, 1, G.stream())
        assert not G.host(wz).any()
    # the dense path on the same data gives the same bits (both sum in ascending feature order)
    xh, nf2, ld = G.dense_padded(data)
    x_d = G.dev(xh)
    got = G.get_rows_dense(x_d, ld, n, nf2, sd, x_d, ld, idx_d, m, sd, kt, **prm)
    _check(name, G.host(got), okm.get_rows(idx))


def test_out_of_range_test_features():
    """Test rows with feature ids beyond the SV set's: dropped from the dot, kept in the self dot (kernelmatrix.cpp:290-295,392)."""
    rng = np.random.default_rng(3)
    sv = from_dense(rng.standard_normal((50, 6)).astype(np.float32))
    tst = from_dense(rng.standard_normal((20, 9)).astype(np.float32))
    p = O.make_param(kernel_type=O.RBF, gamma=0.3, expf_mode=1)
    okm = O.KernelMatrix(sv.ptr, sv.col, sv.val, p)
    want = okm.get_rows_instances(tst.ptr, tst.col, tst.val)
    xh, nf, ld = G.dense_padded(sv)
    x_d = G.dev(xh)
    sd = torch.empty(sv.n, dtype=torch.float64, device="cuda")
    capi.call("tsvm_dense_self_dot", G.ptr(x_d), ld, sv.n, nf, G.ptr(sd), G.stream())
    # batch: CSR -> dense (columns >= ld dropped), self dot over the full CSR row
    val_d, col_d, ptr_d = G.dev(tst.val), G.dev(tst.col), G.dev(tst.ptr)
    b_d = torch.empty((tst.n, ld), dtype=torch.float64, device="cuda")
    capi.call("tsvm_csr_to_dense", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), tst.n, G.ptr(b_d), ld, G.stream())
    b_d[:, nf:] = 0
    sdb = torch.empty(tst.n, dtype=torch.float64, device="cuda")
    capi.call("tsvm_csr_self_dot", G.ptr(val_d), G.ptr(ptr_d), tst.n, G.ptr(sdb), G.stream())
    got = G.get_rows_dense(x_d, ld, sv.n, nf, sd, b_d, ld, None, tst.n, sdb, O.RBF, gamma=0.3)
    assert np.array_equal(G.host(got), want)


@pytest.mark.parametrize("n_classes,rows", [(2, 5), (3, 150), (7, 333), (33, 9), (100, 6)])
def test_sum_kernel_values(n_classes, rows):
    rng = np.random.default_rng(n_classes)
    cnt = rng.integers(1, 300 if n_classes <= 32 else 40, size=n_classes).astype(np.int32)
    if n_classes == 7:
        cnt[3] = 0
    start = np.concatenate([[0], np.cumsum(cnt)[:-1]]).astype(np.int32)
    T = int(cnt.sum())
    coef = rng.standard_normal((n_classes - 1, T))
    nb = n_classes * (n_classes - 1) // 2
    rho = rng.standard_normal(nb)
    k = rng.random((rows, T))
    want = O.sum_kernel_values(coef, T, start, cnt, rho, k, n_classes, rows)
    dec = torch.empty((rows, nb), dtype=torch.float64, device="cuda")
    coef_d, start_d, cnt_d, rho_d, k_d = G.dev(coef), G.dev(start), G.dev(cnt), G.dev(rho), G.dev(k)
    capi.call("tsvm_sum_kernel_values", G.ptr(coef_d), T, G.ptr(start_d), G.ptr(cnt_d), G.ptr(rho_d), G.ptr(k_d),
              capi.ROW_F64, T, G.ptr(dec), n_classes, rows, G.stream())
    assert np.abs(G.host(dec) - want).max() < 1e-9
    # float kernel values: same reduction on the float-rounded matrix
    k32 = k.astype(np.float32)
    want32 = O.sum_kernel_values(coef, T, start, cnt, rho, k32.astype(np.float64), n_classes, rows)
    k32_d = G.dev(k32)
    capi.call("tsvm_sum_kernel_values", G.ptr(coef_d), T, G.ptr(start_d), G.ptr(cnt_d), G.ptr(rho_d), G.ptr(k32_d),
              capi.ROW_F32, T, G.ptr(dec), n_classes, rows, G.stream())
    assert np.abs(G.host(dec) - want32).max() < 1e-9


def test_output_row_slots():
    """get_rows writes row i to out[out_slots[i]] (dense and CSR kernels)."""
    rng = np.random.default_rng(21)
    n, d, m, pool = 300, 20, 40, 64
    data = from_dense(rng.standard_normal((n, d)).astype(np.float32))
    p = O.make_param(kernel_type=O.RBF, gamma=0.2, expf_mode=1)
    want = O.KernelMatrix(data.ptr, data.col, data.val, p).get_rows(np.arange(m))
    x_d, nf, ld, sd, diag = _device_km(data, O.RBF, dict(gamma=0.2))
    slots = rng.permutation(pool)[:m].astype(np.int32)
    idx_d, slots_d = G.dev(np.arange(m, dtype=np.int32)), G.dev(slots)
    got = G.host(G.get_rows_dense(x_d, ld, n, nf, sd, x_d, ld, idx_d, m, sd, O.RBF, gamma=0.2, out_slots=slots_d, out_rows=pool))
    assert np.array_equal(got[slots], want)
    val_d, col_d, ptr_d = G.dev(data.val), G.dev(data.col), G.dev(data.ptr)
    w = torch.empty((nf, m), dtype=torch.float64, device="cuda")
    capi.call("tsvm_csr_stage_rows", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), G.ptr(idx_d), m, nf, G.ptr(w), G.stream())
    sdw = torch.empty(m, dtype=torch.float64, device="cuda")
    capi.call("tsvm_gather_f64", G.ptr(sd), G.ptr(idx_d), m, G.ptr(sdw), G.stream())
    out = torch.zeros((pool, n), dtype=torch.float64, device="cuda")
    capi.call("tsvm_get_rows_csr", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), None, n, G.ptr(sd), G.ptr(w), m, G.ptr(sdw), O.RBF,
              0.2, 0.0, 3, G.ptr(out), capi.ROW_F64, G.ptr(slots_d), n, G.stream())
    assert np.array_equal(G.host(out)[slots], want)


def test_row_subsets_on_device():
    """tsvm_gather_rows_f64 / tsvm_csr_gather_rows: a class pair's rows taken from the resident data set."""
    rng = np.random.default_rng(5)
    n, d, m = 300, 21, 120
    x = rng.standard_normal((n, d)).astype(np.float32)
    x[rng.random((n, d)) < 0.6] = 0
    x[7] = 0                                     # an empty row
    data = from_dense(x)
    idx = rng.permutation(n)[:m].astype(np.int32)
    idx[3] = 7
    xh, nf, ld = G.dense_padded(data)
    x_d, idx_d = G.dev(xh), G.dev(idx)
    out = torch.empty((m, ld), dtype=torch.float64, device="cuda")
    capi.call("tsvm_gather_rows_f64", G.ptr(x_d), ld, G.ptr(idx_d), m, G.ptr(out), G.stream())
    assert np.array_equal(G.host(out), xh[idx])
    sub = data.rows(idx)
    val_d, col_d, ptr_d, optr_d = G.dev(data.val), G.dev(data.col), G.dev(data.ptr), G.dev(sub.ptr)
    oval = torch.empty(sub.nnz, dtype=torch.float64, device="cuda")
    ocol = torch.empty(sub.nnz, dtype=torch.int32, device="cuda")
    capi.call("tsvm_csr_gather_rows", G.ptr(val_d), G.ptr(col_d), G.ptr(ptr_d), G.ptr(idx_d), m, G.ptr(optr_d), G.ptr(oval),
              G.ptr(ocol), G.stream())
    assert np.array_equal(G.host(oval), sub.val) and np.array_equal(G.host(ocol), sub.col)


@pytest.mark.parametrize("n,d,m", [(131072 + 77, 7, 133), (140001, 54, 512), (131072, 90, 200), (135000, 200, 1024), (133333, 16, 65),
                                   (131072 + 5, 24, 100), (131333, 33, 70)])   # one, two, three and more K tiles of 16 columns
def test_dense_rbf_many_columns_few_features(n, d, m):
    """The shapes of the multi-class and regression workloads (hundreds of thousands of columns, tens of features):
    float and double rows, output slots, ragged last tiles in both directions."""
    rng = np.random.default_rng(n + d)
    x = rng.standard_normal((n, d)).astype(np.float32)
    x[rng.random((n, d)) < 0.3] = 0
    data = from_dense(x)
    prm = dict(gamma=0.7 / d)
    p = O.make_param(kernel_type=O.RBF, expf_mode=1, **prm)
    okm = O.KernelMatrix(data.ptr, data.col, data.val, p)
    x_d, nf, ld, sd, diag = _device_km(data, O.RBF, prm)
    idx = rng.integers(0, n, size=m).astype(np.int32)
    idx[-1] = n - 1
    want = okm.get_rows(idx)
    idx_d = G.dev(idx)
    got = G.host(G.get_rows_dense(x_d, ld, n, nf, sd, x_d, ld, idx_d, m, sd, O.RBF, **prm))
    assert np.array_equal(got, want)
    slots = rng.permutation(m + 9)[:m].astype(np.int32)
    got32 = G.host(G.get_rows_dense(x_d, ld, n, nf, sd, x_d, ld, idx_d, m, sd, O.RBF, row_type=capi.ROW_F32,
                                    out_slots=G.dev(slots), out_rows=m + 9, **prm))
    assert np.array_equal(got32[slots].astype(np.float64), want)


@pytest.mark.parametrize("gamma", [0.5, 0.02, -0.5, -0.01])
def test_rbf_arguments_on_both_sides_of_expf_s_range(gamma):
    """Rows at very different scales: arguments of expf inside its range, in the subnormal results' stretch
    (-104 .. -87.3), below it (the value is 0) and, with a negative gamma, above 88.7 (infinity), mixed within one
    wavefront's stores and in whole tiles of their own; float and double rows, bit for bit."""
    rng = np.random.default_rng(3)
    n, d, m = 1500, 20, 200
    x = rng.standard_normal((n, d)).astype(np.float32)
    scale = np.ones(n, dtype=np.float32)
    scale[rng.random(n) < 0.2] = 3.0
    scale[rng.random(n) < 0.05] = 12.0
    scale[600:900] = 2.5          # whole tiles of mid-range arguments
    scale[900:1200] = 0.05        # and of arguments close to zero
    x *= scale[:, None]
    data = from_dense(x)
    prm = dict(gamma=gamma)
    okm = O.KernelMatrix(data.ptr, data.col, data.val, O.make_param(kernel_type=O.RBF, expf_mode=1, **prm))
    x_d, nf, ld, sd, _ = _device_km(data, O.RBF, prm)
    idx = rng.integers(0, n, size=m).astype(np.int32)
    want = okm.get_rows(idx)
    assert (want == 0).any() or gamma < 0
    assert np.isinf(want).any() or gamma > 0
    tiny = np.float32(1.2e-38)
    assert ((want > 0) & (want < tiny)).any() or gamma < 0 or gamma < 0.1
    for row_type in (capi.ROW_F32, capi.ROW_F64):
        got = G.host(G.get_rows_dense(x_d, ld, n, nf, sd, x_d, ld, G.dev(idx), m, sd, O.RBF, row_type=row_type, **prm))
        assert np.array_equal(got.astype(np.float64), want)


@pytest.mark.parametrize("n,d,ws", [(300, 20, 64), (5000, 54, 1024), (2600, 200, 1024)])
def test_row_store_managed_on_the_device(n, d, ws):
    """A row store with a slot for every instance, run the way the solver runs it: tsvm_row_slots_assign decides the
    slots of a working set's new rows, tsvm_get_rows_dense_counted computes exactly those rows into their slots
    (the count stays on the device), tsvm_smo_gather_block_by_id reads the solver's block out of the store.
    Checked against a host-side replay of the bookkeeping, rows from tsvm_get_rows_dense, and the block gathered
    from those rows."""
    rng = np.random.default_rng(n + d)
    data = from_dense(rng.standard_normal((n, d)).astype(np.float32).astype(np.float64))
    kt, prm = O.RBF, dict(gamma=0.5)
    x_d, nf, ld, sd, _ = _device_km(data, kt, prm)
    ldo = G.round_up(n, 8)
    all_rows = G.host(G.get_rows_dense(x_d, ld, n, nf, sd, x_d, ld, None, n, sd, kt, row_type=capi.ROW_F32, **prm))
    store = torch.full((n, ldo), -5.0, dtype=torch.float32, device="cuda")
    slot_of = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    state = torch.zeros(2, dtype=torch.int32, device="cuda")
    info = torch.zeros(2, dtype=torch.int32, device="cuda")
    miss_ids = torch.full((ws,), -9, dtype=torch.int32, device="cuda")      # stale entries must never be read
    miss_slots = torch.full((ws,), -9, dtype=torch.int32, device="cuda")
    slots_ws = torch.zeros(ws, dtype=torch.int32, device="cuda")
    ldk = capi.kernel_lib().tsvm_smo_solve_block_ld(ws)
    q = ws // 2
    h_slot_of, used = np.full(n, -1), 0
    ws_ids = rng.permutation(n)[:ws].astype(np.int32)
    for it in range(4 * n // q + 3):
        if it > 0:   # keep the second half, add q ids that are not in the set: half of them new to the store while any are
            rest = rng.permutation(np.setdiff1d(np.arange(n), ws_ids[q:]))
            unseen = rest[h_slot_of[rest] < 0][:q // 2]
            add = np.concatenate([unseen, np.setdiff1d(rest, unseen, assume_unique=True)[:q - len(unseen)]])
            ws_ids = np.concatenate([ws_ids[q:], rng.permutation(add)]).astype(np.int32)
        first_new, n_new = (0, ws) if it == 0 else (q, q)
        new = ws_ids[first_new:]
        want_miss = [int(i) for i in new if h_slot_of[i] < 0]
        for i in want_miss:
            h_slot_of[i] = used
            used += 1
        ids_d = G.dev(ws_ids)
        capi.call("tsvm_row_slots_assign", G.ptr(ids_d) + 4 * first_new, n_new, G.ptr(slot_of), G.ptr(state), G.ptr(miss_ids),
                  G.ptr(miss_slots), G.ptr(ids_d), ws, G.ptr(slots_ws), G.ptr(info), G.stream())
        capi.call("tsvm_get_rows_dense_counted", G.ptr(x_d), ld, None, n, nf, G.ptr(sd), G.ptr(x_d), ld, G.ptr(miss_ids), n_new,
                  G.ptr(state) + 4, G.ptr(sd), kt, prm["gamma"], 0.0, 3, G.ptr(store), capi.ROW_F32, G.ptr(miss_slots), ldo,
                  G.stream())
        assert G.host(state).tolist() == [used, len(want_miss)] and G.host(info).tolist() == [len(want_miss), used]
        assert G.host(miss_ids)[:len(want_miss)].tolist() == want_miss
        assert np.array_equal(G.host(slot_of), h_slot_of)
        assert np.array_equal(G.host(slots_ws), h_slot_of[ws_ids])
        # the block as doubles and as floats (float rows: the same numbers), turn by turn
        bt, bdt = (capi.ROW_F64, torch.float64) if it % 2 else (capi.ROW_F32, torch.float32)
        kws = torch.full((ws, ldk), 3.0, dtype=bdt, device="cuda")
        out_slots = torch.zeros(ws, dtype=torch.int32, device="cuda")
        capi.call("tsvm_smo_gather_block_by_id", G.ptr(store), capi.ROW_F32, G.ptr(slot_of), ldo, G.ptr(ids_d), ws, G.ptr(kws),
                  bt, G.ptr(out_slots), G.stream())
        got = G.host(kws).astype(np.float64)
        assert np.array_equal(got[:, :ws], all_rows[np.ix_(ws_ids, ws_ids)].astype(np.float64)) and (got[:, ws:] == 0).all()
        assert np.array_equal(G.host(out_slots), h_slot_of[ws_ids])
    assert used == n                                       # every instance has been seen: the store is complete
    st = G.host(store)
    assert np.array_equal(st[h_slot_of][:, :n], all_rows)  # each row computed into its slot, nothing else touched


@pytest.mark.parametrize("name,kt,prm", KERNELS)
@pytest.mark.parametrize("n,d,ws", [(300, 20, 64), (3000, 54, 1000), (2600, 200, 1024), (1500, 784, 200)])
def test_working_set_block(name, kt, prm, n, d, ws):
    """The solver's ws x ws block (x_idx = a_idx = the working set): the same bits as the corresponding entries of the
    full kernel rows, although only the tiles on and above the diagonal are computed and the rest is mirrored."""
    rng = np.random.default_rng(n + ws)
    data = from_dense(rng.standard_normal((n, d)).astype(np.float32).astype(np.float64))
    x_d, nf, ld, sd, _ = _device_km(data, kt, prm)
    ids = rng.permutation(n)[:ws].astype(np.int32)
    if ws >= 8: ids[5] = ids[2]                     # the same row twice (a folded problem can select both copies)
    ids_d = G.dev(ids)
    rows = G.host(G.get_rows_dense(x_d, ld, n, nf, sd, x_d, ld, ids_d, ws, sd, kt, **prm))       # [ws, n]
    ldk = G.round_up(ws, 256)
    blk = torch.full((ws, ldk), 9.0, dtype=torch.float64, device="cuda")
    capi.call("tsvm_get_rows_dense", G.ptr(x_d), ld, G.ptr(ids_d), ws, nf, G.ptr(sd), G.ptr(x_d), ld, G.ptr(ids_d), ws, G.ptr(sd),
              kt, prm.get("gamma", 0.0), prm.get("coef0", 0.0), prm.get("degree", 3), G.ptr(blk), capi.ROW_F64, None, ldk,
              G.stream())
    got = G.host(blk)
    assert np.array_equal(got[:, :ws], rows[:, ids])
    assert np.array_equal(got[:, :ws], got[:, :ws].T)
    assert (got[:, ws:] == 9.0).all()
    if kt != O.LINEAR:      # kernel values that are floats by definition: the block as float elements holds the same numbers
        blk32 = torch.full((ws, ldk), 9.0, dtype=torch.float32, device="cuda")
        capi.call("tsvm_get_rows_dense", G.ptr(x_d), ld, G.ptr(ids_d), ws, nf, G.ptr(sd), G.ptr(x_d), ld, G.ptr(ids_d), ws, G.ptr(sd),
                  kt, prm.get("gamma", 0.0), prm.get("coef0", 0.0), prm.get("degree", 3), G.ptr(blk32), capi.ROW_F32, None, ldk,
                  G.stream())
        got32 = G.host(blk32).astype(np.float64)
        assert np.array_equal(got32[:, :ws], got[:, :ws]) and (got32[:, ws:] == 9.0).all()


def _mixed_rows(rng, n, n_cont, groups):
    """n_cont continuous columns followed by one-hot groups (and, in the last group, rows with no category set)."""
    x = np.zeros((n, n_cont + sum(groups)), dtype=np.float32)
    x[:, :n_cont] = rng.standard_normal((n, n_cont))
    x[:, :n_cont][rng.random((n, n_cont)) < 0.1] = 0
    at = n_cont
    for gi, g in enumerate(groups):
        cat = rng.integers(0, g, n)
        x[np.arange(n), at + cat] = 1
        if gi == len(groups) - 1:
            x[rng.random(n) < 0.05, at:at + g] = 0
        at += g
    return x


@pytest.mark.parametrize("n,n_cont,groups,m", [(140001, 10, (4, 40), 512), (70000, 3, (2, 3, 5, 7), 130), (3000, 0, (6, 10), 64),
                                                (50000, 21, (64,), 200)])
@pytest.mark.parametrize("name,kt,prm", [("rbf", O.RBF, dict(gamma=1.0)), ("linear", O.LINEAR, dict()),
                                         ("poly", O.POLY, dict(gamma=0.3, coef0=0.5, degree=3))])
def test_indicator_columns(n, n_cont, groups, m, name, kt, prm):
    """Trailing 0/1 columns handled by the epilogue (one addition of 1.0 per column set in both rows) instead of the
    matrix cores: the same bits as the plain kernel and the oracle, for every kernel, float and double rows, output
    slots, a device-side row count and a column subset."""
    rng = np.random.default_rng(n + n_cont)
    x = _mixed_rows(rng, n, n_cont, groups)
    data = from_dense(x)
    p = O.make_param(kernel_type=kt, expf_mode=1, **prm)
    okm = O.KernelMatrix(data.ptr, data.col, data.val, p)
    x_d, nf, ld, sd, diag = _device_km(data, kt, prm)
    first = 1 + n_cont                                    # column 0 is the unused feature id 0
    n_ind = nf - first
    masks = torch.zeros(n, dtype=torch.int64, device="cuda")
    max_ones = torch.full((1,), -7, dtype=torch.int32, device="cuda")
    capi.call("tsvm_indicator_masks", G.ptr(x_d), ld, n, first, n_ind, G.ptr(masks), G.ptr(max_ones), G.stream())
    want_mask = (x[:, n_cont:] != 0).astype(np.uint64) @ (np.uint64(1) << np.arange(n_ind, dtype=np.uint64))
    assert np.array_equal(G.host(masks).view(np.uint64), want_mask)
    mo = int(G.host(max_ones)[0])
    assert mo == int((x[:, n_cont:] != 0).sum(axis=1).max()) == len(groups)
    idx = rng.integers(0, n, size=m).astype(np.int32)
    idx[-1] = n - 1
    want = okm.get_rows(idx)
    idx_d = G.dev(idx)
    g = prm.get("gamma", 0.0), prm.get("coef0", 0.0), prm.get("degree", 3)

    def run(row_type, out, m_run, m_dev=None, slots=None, x_idx=None, n_cols=n):
        capi.call("tsvm_get_rows_dense_indicator", G.ptr(x_d), ld, G.ptr(x_idx), n_cols, first, G.ptr(sd), G.ptr(masks), G.ptr(x_d),
                  ld, G.ptr(idx_d), m_run, G.ptr(m_dev), G.ptr(sd), G.ptr(masks), mo, kt, *g, G.ptr(out), row_type,
                  G.ptr(slots), out.shape[1], G.stream())

    out = torch.full((m, n), -3.0, dtype=torch.float64, device="cuda")
    run(capi.ROW_F64, out, m)
    _check(name, G.host(out), want)
    if kt != O.LINEAR:
        # float rows into permuted slots, the row count read on the device (grid sized for more rows)
        slots = rng.permutation(m + 9)[:m].astype(np.int32)
        out32 = torch.full((m + 9, n), -3.0, dtype=torch.float32, device="cuda")
        m_dev = G.dev(np.array([m - 5], dtype=np.int32))
        run(capi.ROW_F32, out32, m, m_dev=m_dev, slots=G.dev(slots))
        got = G.host(out32)
        _check(name, got[slots[:m - 5]].astype(np.float64), want[:m - 5])
        assert (got[slots[m - 5:]] == -3.0).all()
    # a column subset (the solver's block shape)
    cols = rng.permutation(n)[:777].astype(np.int32)
    outb = torch.empty((m, 777), dtype=torch.float64, device="cuda")
    run(capi.ROW_F64, outb, m, x_idx=G.dev(cols), n_cols=777)
    _check(name, G.host(outb), want[:, cols])
