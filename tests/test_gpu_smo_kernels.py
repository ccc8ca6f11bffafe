"""GPU parity: update_f, c_smo_solve, nu_smo_solve and the fused sort_f + select_working_set
through the C ABI vs the CPU oracle.  All bit-exact / index-exact."""
import numpy as np
import pytest
import torch

import gpu_util as G
import oracle_lib as O
from thundersvm_amd import capi
from thundersvm_amd.data import from_dense

pytestmark = pytest.mark.gpu


def _problem(n, d, seed, gamma=0.5):
    rng = np.random.default_rng(seed)
    y = np.where(rng.random(n) < 0.5, 1, -1).astype(np.int32)
    x = (rng.standard_normal((n, d)) + 0.4 * y[:, None]).astype(np.float32)
    data = from_dense(x)
    p = O.make_param(kernel_type=O.RBF, gamma=gamma, expf_mode=1)
    km = O.KernelMatrix(data.ptr, data.col, data.val, p)
    return rng, y, km


@pytest.mark.parametrize("n,ws,zero_frac", [(1, 1, 0.0), (1000, 1024, 0.5), (1537, 512, 0.0), (4099, 37, 0.9), (513, 2050, 0.3)])
@pytest.mark.parametrize("row_type", [capi.ROW_F64, capi.ROW_F32])
def test_update_f(n, ws, zero_frac, row_type):
    rng = np.random.default_rng(n + ws)
    ld = n + 3
    k = rng.random((ws + 5, ld))
    if row_type == capi.ROW_F32:
        k = k.astype(np.float32)
    k64 = k.astype(np.float64)
    ad = rng.standard_normal(ws)
    ad[rng.random(ws) < zero_frac] = 0
    f = rng.standard_normal(n)
    slots = rng.permutation(ws + 5)[:ws].astype(np.int32)
    want = O.update_f(f, ad, np.ascontiguousarray(k64[slots][:, :n]), n)
    f_d, ad_d, k_d, s_d = G.dev(f), G.dev(ad), G.dev(k), G.dev(slots)
    capi.call("tsvm_update_f", G.ptr(f_d), G.ptr(ad_d), ws, G.ptr(k_d), row_type, G.ptr(s_d), ld, n, 1, G.stream())
    assert np.array_equal(G.host(f_d), want)
    # slots == NULL: identity
    want = O.update_f(f, ad, np.ascontiguousarray(k64[:ws, :n]), n)
    f_d = G.dev(f)
    capi.call("tsvm_update_f", G.ptr(f_d), G.ptr(ad_d), ws, G.ptr(k_d), row_type, None, ld, n, 1, G.stream())
    assert np.array_equal(G.host(f_d), want)


@pytest.mark.parametrize("n,ws,ld_pad", [(300001, 64, 7), (262144, 33, 0), (270000, 40, 4)])
@pytest.mark.parametrize("row_type", [capi.ROW_F64, capi.ROW_F32])
def test_update_f_wide_and_repeated(n, ws, ld_pad, row_type):
    """Large n takes the 16-byte-load path (also with a ragged last vector); with repeat = 2 the kernel
    rows are n wide and f has 2n entries, which must equal the reference's update_f on [K K] rows."""
    rng = np.random.default_rng(n)
    ld = n + ld_pad
    k = rng.random((ws, ld))
    if row_type == capi.ROW_F32:
        k = k.astype(np.float32)
    k64 = k.astype(np.float64)[:, :n]
    ad = rng.standard_normal(ws)
    ad[::3] = 0
    f = rng.standard_normal(2 * n)
    want = O.update_f(f, ad, np.ascontiguousarray(np.concatenate([k64, k64], axis=1)), 2 * n)
    f_d, ad_d, k_d = G.dev(f), G.dev(ad), G.dev(k)
    capi.call("tsvm_update_f", G.ptr(f_d), G.ptr(ad_d), ws, G.ptr(k_d), row_type, None, ld, n, 2, G.stream())
    assert np.array_equal(G.host(f_d), want)


def test_fold_ids():
    ids = np.array([0, 5, 9, 10, 19, 7], dtype=np.int32)
    out = torch.zeros(6, dtype=torch.int32, device="cuda")
    ids_d = G.dev(ids)
    capi.call("tsvm_fold_ids", G.ptr(ids_d), 6, 10, G.ptr(out), G.stream())
    assert np.array_equal(G.host(out), ids % 10)


def _solver_inputs(n, d, ws, seed, C, nu=False):
    rng, y, km = _problem(n, d, seed)
    alpha = np.zeros(n)
    # a mid-training state: some alphas at bounds, some free
    r = rng.random(n)
    alpha[r < 0.2] = C
    alpha[(r >= 0.2) & (r < 0.5)] = rng.random(int(((r >= 0.2) & (r < 0.5)).sum())) * C
    f = rng.standard_normal(n)
    ws_ids = rng.permutation(n)[:ws].astype(np.int32)
    k_rows = km.get_rows(ws_ids)
    diag = km.diag()
    return y, alpha, f, ws_ids, k_rows, diag


@pytest.mark.parametrize("n,ws,max_iter", [(300, 16, 100000), (2000, 1024, 100000), (1500, 512, 7), (700, 100, 100000), (64, 64, 0)])
def test_c_smo_solve(n, ws, max_iter):
    Cp, Cn, eps = 10.0, 4.0, 1e-3
    y, alpha, f, ws_ids, k_rows, diag = _solver_inputs(n, 12, ws, n + ws, Cn)
    a_want, ad_want, diff_want = O.c_smo_solve(y, f, alpha, ws_ids, Cp, Cn, k_rows, diag, n, eps, max_iter)
    slots = np.random.default_rng(1).permutation(ws).astype(np.int32)
    k_phys = np.empty_like(k_rows)
    k_phys[slots] = k_rows
    y_d, f_d, a_d, ws_d, k_d, s_d, dg_d = G.dev(y), G.dev(f), G.dev(alpha), G.dev(ws_ids), G.dev(k_phys), G.dev(slots), G.dev(diag)
    ad_d = torch.zeros(ws, dtype=torch.float64, device="cuda")
    diff_d = torch.zeros(2, dtype=torch.float64, device="cuda")
    wsp = torch.empty(capi.kernel_lib().tsvm_smo_solve_workspace(ws), dtype=torch.uint8, device="cuda")
    capi.call("tsvm_c_smo_solve", G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cp, Cn, G.ptr(k_d),
              capi.ROW_F64, G.ptr(s_d), n, G.ptr(dg_d), eps, G.ptr(diff_d), max_iter, G.ptr(wsp), G.stream())
    assert np.array_equal(G.host(diff_d), diff_want)
    assert np.array_equal(G.host(a_d), a_want)
    assert np.array_equal(G.host(ad_d), ad_want)
    # the same rows held as float (RBF values are float-exact): identical result
    a_d, k32_d = G.dev(alpha), G.dev(k_phys.astype(np.float32))
    assert np.array_equal(k_phys.astype(np.float32).astype(np.float64), k_phys)
    capi.call("tsvm_c_smo_solve", G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cp, Cn, G.ptr(k32_d),
              capi.ROW_F32, G.ptr(s_d), n, G.ptr(dg_d), eps, G.ptr(diff_d), max_iter, G.ptr(wsp), G.stream())
    assert np.array_equal(G.host(diff_d), diff_want)
    assert np.array_equal(G.host(a_d), a_want)
    assert np.array_equal(G.host(ad_d), ad_want)
    assert diff_want[1] > 0 or max_iter == 0 or diff_want[0] < eps


@pytest.mark.parametrize("n,ws", [(300, 16), (2000, 1024), (900, 200)])
def test_nu_smo_solve(n, ws):
    Cc, eps = 1.0, 1e-3
    y, alpha, f, ws_ids, k_rows, diag = _solver_inputs(n, 10, ws, 5 * n + ws, Cc)
    a_want, ad_want, diff_want = O.nu_smo_solve(y, f, alpha, ws_ids, Cc, k_rows, diag, n, eps, 100000)
    y_d, f_d, a_d, ws_d, k_d, dg_d = G.dev(y), G.dev(f), G.dev(alpha), G.dev(ws_ids), G.dev(k_rows), G.dev(diag)
    ad_d = torch.zeros(ws, dtype=torch.float64, device="cuda")
    diff_d = torch.zeros(2, dtype=torch.float64, device="cuda")
    wsp = torch.empty(capi.kernel_lib().tsvm_smo_solve_workspace(ws), dtype=torch.uint8, device="cuda")
    capi.call("tsvm_nu_smo_solve", G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cc, G.ptr(k_d),
              capi.ROW_F64, None, n, G.ptr(dg_d), eps, G.ptr(diff_d), 100000, G.ptr(wsp), G.stream())
    assert G.host(diff_d)[0] == diff_want[0]
    assert np.array_equal(G.host(a_d), a_want)
    assert np.array_equal(G.host(ad_d), ad_want)
    # the same rows held as float: a float block inside, identical result
    a_d, k32_d = G.dev(alpha), G.dev(k_rows.astype(np.float32))
    capi.call("tsvm_nu_smo_solve", G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cc, G.ptr(k32_d),
              capi.ROW_F32, None, n, G.ptr(dg_d), eps, G.ptr(diff_d), 100000, G.ptr(wsp), G.stream())
    assert G.host(diff_d)[0] == diff_want[0]
    assert np.array_equal(G.host(a_d), a_want)
    assert np.array_equal(G.host(ad_d), ad_want)


@pytest.mark.parametrize("nu", [False, True])
@pytest.mark.parametrize("n,ws", [(300, 16), (2000, 1024), (900, 200)])
def test_smo_solve_block_on_a_chosen_xcd(n, ws, nu):
    """The block solvers launched as eight workgroups of which one is elected (tsvm_*_smo_solve_block_on_xcd): the same
    result as the one-workgroup launch, for every target XCD and launch after launch on one gate.  On an ordinary
    stream the eight workgroups land wherever there is room, so some targets have a workgroup on them and others
    do not: both ways of being elected (being on the target, being the last to arrive) are exercised, and exactly one
    workgroup solves either way (two would apply every step twice)."""
    Cc, eps = 1.0, 1e-3
    y, alpha, f, ws_ids, k_rows, diag = _solver_inputs(n, 10, ws, 7 * n + ws, Cc, nu)
    if nu:
        a_want, ad_want, diff_want = O.nu_smo_solve(y, f, alpha, ws_ids, Cc, k_rows, diag, n, eps, 100000)
    else:
        a_want, ad_want, diff_want = O.c_smo_solve(y, f, alpha, ws_ids, Cc, Cc, k_rows, diag, n, eps, 100000)
    ldk = capi.kernel_lib().tsvm_smo_solve_block_ld(ws)
    block = np.zeros((ws, ldk))
    block[:, :ws] = k_rows[:, ws_ids]
    y_d, f_d, ws_d, b_d, dg_d = G.dev(y), G.dev(f), G.dev(ws_ids), G.dev(block), G.dev(diag)
    assert np.array_equal(block.astype(np.float32).astype(np.float64), block)     # RBF values: a float block holds the same numbers
    b32_d = G.dev(block.astype(np.float32))
    gate = torch.zeros(4, dtype=torch.int32, device="cuda")
    seen = set()
    for epoch, xcd in enumerate([0, 3, 7, 5, 1, 2, 6, 4, 0, 0], start=1):
        a_d = G.dev(alpha)
        ad_d = torch.zeros(ws, dtype=torch.float64, device="cuda")
        diff_d = torch.zeros(2, dtype=torch.float64, device="cuda")
        blk, bt = (b_d, capi.ROW_F64) if epoch % 2 else (b32_d, capi.ROW_F32)
        if nu:
            capi.call("tsvm_nu_smo_solve_block_on_xcd", G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cc,
                      G.ptr(blk), bt, G.ptr(dg_d), eps, G.ptr(diff_d), 100000, G.ptr(gate), epoch, xcd, G.stream())
        else:
            capi.call("tsvm_c_smo_solve_block_on_xcd", G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cc, Cc,
                      G.ptr(blk), bt, G.ptr(dg_d), eps, G.ptr(diff_d), 100000, G.ptr(gate), epoch, xcd, G.stream())
        g = G.host(gate)
        assert g[0] == epoch and g[1] == 8 * epoch and 0 <= g[2] < 8
        seen.add(int(g[2]))
        assert G.host(diff_d)[0] == diff_want[0]
        assert np.array_equal(G.host(a_d), a_want)
        assert np.array_equal(G.host(ad_d), ad_want)
    # bad arguments are refused
    lib = capi.kernel_lib()
    assert lib.tsvm_c_smo_solve_block_on_xcd(G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cc, Cc, G.ptr(b_d),
                                             capi.ROW_F64, G.ptr(dg_d), eps, G.ptr(diff_d), 10, G.ptr(gate), 0, 0, G.stream()) != 0
    assert lib.tsvm_c_smo_solve_block_on_xcd(G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cc, Cc, G.ptr(b_d),
                                             capi.ROW_F64, G.ptr(dg_d), eps, G.ptr(diff_d), 10, G.ptr(gate), 1, 8, G.stream()) != 0
    assert lib.tsvm_c_smo_solve_block_on_xcd(G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cc, Cc, G.ptr(b_d),
                                             7, G.ptr(dg_d), eps, G.ptr(diff_d), 10, G.ptr(gate), 1, 0, G.stream()) != 0


def _select_case(n, n_select, n_marked, seed, tie_mode, nu):
    rng = np.random.default_rng(seed)
    y = np.where(rng.random(n) < 0.5, 1, -1).astype(np.int32)
    C = 2.0
    alpha = np.zeros(n)
    r = rng.random(n)
    alpha[r < 0.25] = C
    free = (r >= 0.25) & (r < 0.5)
    alpha[free] = rng.random(int(free.sum())) * C
    if tie_mode == 0:
        f = rng.standard_normal(n)
    elif tie_mode == 1:
        f = -y.astype(np.float64)               # the initial state of C-SVC: massive ties
    else:
        f = np.round(rng.standard_normal(n), 1)  # few distinct values, signed zeros
        f[rng.random(n) < 0.1] = -0.0
    marked = rng.permutation(n)[:n_marked].astype(np.int32)
    return f, y, alpha, C, marked


@pytest.mark.parametrize("nu", [0, 1])
@pytest.mark.parametrize("tie_mode", [0, 1, 2])
@pytest.mark.parametrize("n,n_select,n_marked", [(2, 2, 0), (150, 128, 0), (150, 64, 64), (3200, 1024, 0), (3200, 512, 512),
                                                 (100000, 512, 512), (70001, 1024, 0), (1100, 1024, 0), (1030, 512, 512),
                                                 (1200000, 512, 512)])
def test_select_working_set(n, n_select, n_marked, tie_mode, nu):
    f, y, alpha, C, marked = _select_case(n, n_select, n_marked, n + n_select + tie_mode, tie_mode, nu)
    want = O.select_working_set(f, y, alpha, C, C, marked, n_select, nu=bool(nu))
    f_d, y_d, a_d, m_d = G.dev(f), G.dev(y), G.dev(alpha), G.dev(marked)
    out_d = torch.full((n_select,), -7, dtype=torch.int32, device="cuda")
    wsp = torch.empty(capi.kernel_lib().tsvm_select_workspace(n), dtype=torch.uint8, device="cuda")
    capi.call("tsvm_select_working_set", G.ptr(f_d), G.ptr(y_d), G.ptr(a_d), n, C, C, G.ptr(m_d) if n_marked else None,
              n_marked, G.ptr(out_d), n_select, nu, G.ptr(wsp), G.stream())
    got = G.host(out_d)
    assert np.array_equal(got, want), "first mismatch at %s" % np.flatnonzero(got != want)[:5]


@pytest.mark.parametrize("nu", [0, 1])
@pytest.mark.parametrize("tie_mode", [0, 1, 2])
def test_longer_selection_starts_with_the_shorter_one(tie_mode, nu):
    """Asking for more ids appends runners-up: the first n_select ids do not change."""
    n, n_marked = 50000, 512
    f, y, alpha, C, marked = _select_case(n, 512, n_marked, 99 + tie_mode, tie_mode, nu)
    f_d, y_d, a_d, m_d = G.dev(f), G.dev(y), G.dev(alpha), G.dev(marked)
    wsp = torch.empty(capi.kernel_lib().tsvm_select_workspace(n), dtype=torch.uint8, device="cuda")
    outs = []
    for n_select in (512, 768):
        out_d = torch.full((n_select,), -7, dtype=torch.int32, device="cuda")
        capi.call("tsvm_select_working_set", G.ptr(f_d), G.ptr(y_d), G.ptr(a_d), n, C, C, G.ptr(m_d), n_marked, G.ptr(out_d),
                  n_select, nu, G.ptr(wsp), G.stream())
        outs.append(G.host(out_d))
    assert np.array_equal(outs[1][:512], outs[0])
    assert np.array_equal(outs[1], O.select_working_set(f, y, alpha, C, C, marked, 768, nu=bool(nu)))
    tail = outs[1][512:]
    assert (tail >= 0).all() and len(set(tail.tolist()) | set(outs[0].tolist()) | set(marked.tolist())) == 768 + n_marked


@pytest.mark.parametrize("nu", [0, 1])
@pytest.mark.parametrize("n", [700, 3200, 100000, 300001])
def test_selections_in_a_row_on_one_workspace(n, nu):
    """The solver's pattern (csmosolver.cpp:63-77): one full selection, then one per outer iteration that keeps
    half of the previous set, all on one workspace that each call leaves ready for the next.  The f values change
    from call to call between distinct values, massive ties (the remaining digits are then resolved by the final
    kernel's workgroup) and few distinct values."""
    ws = min(1024, 1 << (n.bit_length() - 1))
    q = ws // 2
    wsp = torch.empty(capi.kernel_lib().tsvm_select_workspace(n), dtype=torch.uint8, device="cuda")
    wsp.random_(0, 256)   # whatever an earlier user of the memory left there
    prev = None
    for it, tie_mode in enumerate([0, 1, 0, 2, 1, 1, 0]):
        f, y, alpha, C, _ = _select_case(n, q, 0, 7 * n + it, tie_mode, nu)
        marked = np.zeros(0, dtype=np.int32) if it == 0 else np.ascontiguousarray(prev[q:])
        n_select = ws if it == 0 else q
        want = O.select_working_set(f, y, alpha, C, C, marked, n_select, nu=bool(nu))
        f_d, y_d, a_d, m_d = G.dev(f), G.dev(y), G.dev(alpha), G.dev(marked if it else np.zeros(1, dtype=np.int32))
        out_d = torch.full((n_select,), -7, dtype=torch.int32, device="cuda")
        capi.call("tsvm_select_working_set" if it == 0 else "tsvm_select_working_set_again", G.ptr(f_d), G.ptr(y_d),
                  G.ptr(a_d), n, C, C, G.ptr(m_d) if it else None, len(marked), G.ptr(out_d), n_select, nu, G.ptr(wsp),
                  G.stream())
        got = G.host(out_d)
        assert np.array_equal(got, want), "call %d: first mismatch at %s" % (it, np.flatnonzero(got != want)[:5])
        prev = got if it == 0 else np.concatenate([prev[q:], got])
        assert (prev >= 0).all()


@pytest.mark.parametrize("nu", [0, 1])
@pytest.mark.parametrize("n,tie_mode", [(150, 0), (5000, 2), (200000, 0), (200000, 1)])
def test_selection_with_folded_ids(n, tie_mode, nu):
    """The 2n-variable problem of SVR (svr.cpp:14-28): the selection also delivers each id modulo n / 2, the stored row
    behind the variable; same ids as the plain selection, on a fresh and on a re-used workspace."""
    half = n // 2
    ws = min(1024, 1 << (n.bit_length() - 1))
    q = ws // 2
    wsp = torch.empty(capi.kernel_lib().tsvm_select_workspace(n), dtype=torch.uint8, device="cuda")
    prev = None
    for it in range(3):
        f, y, alpha, C, _ = _select_case(n, q, 0, 5 * n + it, tie_mode, nu)
        marked = np.zeros(0, dtype=np.int32) if it == 0 else np.ascontiguousarray(prev[q:])
        n_select = ws if it == 0 else q
        want = O.select_working_set(f, y, alpha, C, C, marked, n_select, nu=bool(nu))
        f_d, y_d, a_d, m_d = G.dev(f), G.dev(y), G.dev(alpha), G.dev(marked if it else np.zeros(1, dtype=np.int32))
        out_d = torch.full((n_select,), -7, dtype=torch.int32, device="cuda")
        fold_d = torch.full((n_select,), -7, dtype=torch.int32, device="cuda")
        capi.call("tsvm_select_working_set_folded", G.ptr(f_d), G.ptr(y_d), G.ptr(a_d), n, C, C, G.ptr(m_d) if it else None,
                  len(marked), G.ptr(out_d), n_select, nu, G.ptr(wsp), int(it > 0), half, G.ptr(fold_d), G.stream())
        got = G.host(out_d)
        assert np.array_equal(got, want)
        assert np.array_equal(G.host(fold_d), np.where(want >= 0, want % half, -1))
        prev = got if it == 0 else np.concatenate([prev[q:], got])


@pytest.mark.parametrize("nu", [0, 1])
@pytest.mark.parametrize("row_type", [capi.ROW_F64, capi.ROW_F32])
@pytest.mark.parametrize("n_cols,repeat,ws,ld_pad,tie_mode", [(1, 1, 1, 0, 0), (700, 1, 512, 3, 0), (4099, 2, 64, 1, 2),
                                                             (300001, 1, 1024, 7, 0), (270000, 2, 200, 0, 0),
                                                             (262144, 1, 1024, 0, 1), (150000, 3, 16, 4, 2)])
def test_update_f_with_the_next_selection(n_cols, repeat, ws, ld_pad, tie_mode, row_type, nu):
    """One call that updates f and selects the next working set on the new values: f as the oracle's update_f leaves
    it, the ids as the oracle's selection on that f, with the half of the previous set that stays excluded.  Two such
    calls in a row on one workspace; with tie_mode 1 and 2 the update changes nothing (all alpha_diff zero), so that
    the selection meets massive ties and few distinct values."""
    n = n_cols * repeat
    rng = np.random.default_rng(n + ws + nu)
    ld = n_cols + ld_pad
    k = rng.random((ws, ld))
    if row_type == capi.ROW_F32:
        k = k.astype(np.float32)
    k64 = np.ascontiguousarray(np.concatenate([k.astype(np.float64)[:, :n_cols]] * repeat, axis=1))
    sel = min(1024, 1 << (n.bit_length() - 1))
    q = max(sel // 2, 1)
    f, y, alpha, C, _ = _select_case(n, q, 0, 3 * n + 1, tie_mode, nu)
    f_d, y_d, a_d, k_d = G.dev(f), G.dev(y), G.dev(alpha), G.dev(k)
    wsp = torch.empty(capi.kernel_lib().tsvm_select_workspace(n), dtype=torch.uint8, device="cuda")
    wsp.random_(0, 256)
    out_d = torch.full((sel,), -7, dtype=torch.int32, device="cuda")
    capi.call("tsvm_select_working_set", G.ptr(f_d), G.ptr(y_d), G.ptr(a_d), n, C, C, None, 0, G.ptr(out_d), sel, nu, G.ptr(wsp),
              G.stream())
    prev = G.host(out_d)
    assert np.array_equal(prev, O.select_working_set(f, y, alpha, C, C, np.zeros(0, dtype=np.int32), sel, nu=bool(nu)))
    for call in range(2):
        marked = np.ascontiguousarray(prev[sel - q:]) if sel > 1 else np.zeros(0, dtype=np.int32)
        marked = marked[marked >= 0]
        ad = rng.standard_normal(ws)
        ad[rng.random(ws) < 0.4] = 0
        if tie_mode:
            ad[:] = 0
        f = O.update_f(f, ad, k64, n)
        want = O.select_working_set(f, y, alpha, C, C, marked, q, nu=bool(nu))
        ad_d, m_d = G.dev(ad), G.dev(marked if len(marked) else np.zeros(1, dtype=np.int32))
        new_d = torch.full((q,), -7, dtype=torch.int32, device="cuda")
        folded_d = torch.full((q,), -7, dtype=torch.int32, device="cuda")
        capi.call("tsvm_update_f_select", G.ptr(f_d), G.ptr(ad_d), ws, G.ptr(k_d), row_type, None, ld, n_cols, repeat, G.ptr(y_d),
                  G.ptr(a_d), C, C, G.ptr(m_d) if len(marked) else None, len(marked), G.ptr(new_d), q, nu, G.ptr(wsp),
                  G.ptr(folded_d) if repeat > 1 else None, G.stream())
        assert np.array_equal(G.host(f_d), f)
        got = G.host(new_d)
        assert np.array_equal(got, want), "call %d: first mismatch at %s" % (call, np.flatnonzero(got != want)[:5])
        if repeat > 1:
            assert np.array_equal(G.host(folded_d), np.where(want >= 0, want % n_cols, -1))
        prev = np.concatenate([prev[q:], got]) if sel > 1 else got
        # the instances change their state between the calls, as the local solver would change them
        alpha = alpha.copy()
        alpha[rng.integers(0, n, size=min(n, 300))] = rng.choice([0.0, C, 0.5 * C], size=min(n, 300))
        a_d = G.dev(alpha)


def test_empty_inputs_are_no_ops():
    """Zero rows, zero columns, an empty working set, nothing to select: every entry point returns success and
    leaves its outputs untouched."""
    x = torch.zeros((4, 8), dtype=torch.float64, device="cuda")
    sd = torch.zeros(4, dtype=torch.float64, device="cuda")
    out = torch.full((4, 8), 7.0, dtype=torch.float64, device="cuda")
    for n, m in ((0, 4), (4, 0)):
        capi.call("tsvm_get_rows_dense", G.ptr(x), 8, None, n, 3, G.ptr(sd), G.ptr(x), 8, None, m, G.ptr(sd), 2, 0.5, 0.0, 3,
                  G.ptr(out), capi.ROW_F64, None, 8, G.stream())
    f = torch.full((5,), 3.0, dtype=torch.float64, device="cuda")
    ad = torch.ones(4, dtype=torch.float64, device="cuda")
    capi.call("tsvm_update_f", G.ptr(f), G.ptr(ad), 0, G.ptr(out), capi.ROW_F64, None, 8, 5, 1, G.stream())
    capi.call("tsvm_update_f", G.ptr(f), G.ptr(ad), 4, G.ptr(out), capi.ROW_F64, None, 8, 0, 1, G.stream())
    ids = torch.full((4,), -7, dtype=torch.int32, device="cuda")
    y = torch.ones(5, dtype=torch.int32, device="cuda")
    wsp = torch.empty(capi.kernel_lib().tsvm_select_workspace(5), dtype=torch.uint8, device="cuda")
    capi.call("tsvm_select_working_set", G.ptr(f), G.ptr(y), G.ptr(f), 5, 1.0, 1.0, None, 0, G.ptr(ids), 0, 0, G.ptr(wsp),
              G.stream())
    assert (G.host(out) == 7.0).all() and (G.host(f) == 3.0).all() and (G.host(ids) == -7).all()
    # an all-zero alpha_diff reads no row at all and leaves f as it is
    zeros = torch.zeros(4, dtype=torch.float64, device="cuda")
    capi.call("tsvm_update_f", G.ptr(f), G.ptr(zeros), 4, G.ptr(out), capi.ROW_F64, None, 8, 5, 1, G.stream())
    assert (G.host(f) == 3.0).all()


def test_report_ids_to_host_memory():
    """tsvm_report_ids: the ids land in host memory the device can write, folded when asked, and the word the host polls
    is there once the stream has run (a host-side row store reads its new ids this way instead of through a copy)."""
    rng = np.random.default_rng(4)
    ids = rng.integers(0, 50000, size=512).astype(np.int32)
    ids[7] = -1                                             # a side that ran dry leaves -1
    ids_d = G.dev(ids)
    host = torch.full((1024 + 16,), -7, dtype=torch.int32).pin_memory()
    for n_ids, fold, word in [(512, 0, 1), (512, 20000, 2), (100, 0, 3), (0, 0, 4)]:
        capi.call("tsvm_report_ids", G.ptr(ids_d), n_ids, fold, host.data_ptr(), 1024, word, G.stream())
        torch.cuda.synchronize()
        got = host.numpy()
        want = ids[:n_ids].copy()
        if fold:
            want[want >= 0] %= fold
        assert np.array_equal(got[:n_ids], want) and got[1024] == word
    with pytest.raises(capi.TsvmError):
        capi.call("tsvm_report_ids", G.ptr(ids_d), 600, 0, host.data_ptr(), 512, 1, G.stream())      # the word would lie inside the ids
