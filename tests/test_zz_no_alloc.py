"""tsvm_c_smo_solve_static (the entry point that allocates nothing: its ws x ws block lives in a static device
array) against tsvm_c_smo_solve on the same inputs, bit for bit, on two calls in a row, the second one smaller."""
import numpy as np
import pytest
import torch

import gpu_util as G
from test_gpu_smo_kernels import _solver_inputs
from thundersvm_amd import capi

pytestmark = pytest.mark.gpu


def _both(n, ws, row_type, seed_off, check_device_free=True):
    Cp, Cn, eps, max_iter = 10.0, 4.0, 1e-3, 100000
    y, alpha, f, ws_ids, k_rows, diag = _solver_inputs(n, 12, ws, n + ws + seed_off, Cn)
    slots = np.random.default_rng(seed_off).permutation(ws).astype(np.int32)
    k_phys = np.empty_like(k_rows)
    k_phys[slots] = k_rows
    if row_type == capi.ROW_F32:
        k_phys = k_phys.astype(np.float32)
    y_d, f_d, ws_d, k_d, s_d, dg_d = G.dev(y), G.dev(f), G.dev(ws_ids), G.dev(k_phys), G.dev(slots), G.dev(diag)
    out = []
    for static in (False, True):
        a_d = G.dev(alpha)
        ad_d = torch.zeros(ws, dtype=torch.float64, device="cuda")
        diff_d = torch.zeros(2, dtype=torch.float64, device="cuda")
        if static:
            torch.cuda.synchronize()
            before = torch.cuda.memory_allocated()
            free_before = torch.cuda.mem_get_info()[0]
            capi.call("tsvm_c_smo_solve_static", G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cp, Cn,
                      G.ptr(k_d), row_type, G.ptr(s_d), n, G.ptr(dg_d), eps, G.ptr(diff_d), max_iter, G.stream())
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated() == before
            # (after tsvm_c_smo_solve_static_init nothing is left to look up or load)
            assert not check_device_free or torch.cuda.mem_get_info()[0] == free_before
        else:
            wsp = torch.empty(capi.kernel_lib().tsvm_smo_solve_workspace(ws), dtype=torch.uint8, device="cuda")
            capi.call("tsvm_c_smo_solve", G.ptr(y_d), G.ptr(f_d), G.ptr(a_d), G.ptr(ad_d), G.ptr(ws_d), ws, Cp, Cn,
                      G.ptr(k_d), row_type, G.ptr(s_d), n, G.ptr(dg_d), eps, G.ptr(diff_d), max_iter, G.ptr(wsp), G.stream())
        out.append((G.host(a_d).copy(), G.host(ad_d).copy(), G.host(diff_d).copy()))
    (a0, ad0, d0), (a1, ad1, d1) = out
    assert d0[1] > 0
    assert np.array_equal(d0, d1) and np.array_equal(a0, a1) and np.array_equal(ad0, ad1)


def test_static_solver_matches_workspace_solver_twice():
    # once per device, outside any capture: the array's address, the kernels' attributes, the code object
    assert capi.kernel_lib().tsvm_c_smo_solve_static_init() == 0, capi.kernel_lib().tsvm_last_error()
    _both(2000, 1024, capi.ROW_F64, 0)    # fills the whole static block
    _both(700, 100, capi.ROW_F32, 1)      # smaller: reads nothing the first call left behind
    _both(900, 300, capi.ROW_F64, 2)


def test_static_solver_rejects_oversize():
    z = torch.zeros(4096, dtype=torch.float64, device="cuda")
    zi = torch.zeros(4096, dtype=torch.int32, device="cuda")
    rc = capi.kernel_lib().tsvm_c_smo_solve_static(G.ptr(zi), G.ptr(z), G.ptr(z), G.ptr(z), G.ptr(zi), 1025, 1.0, 1.0, G.ptr(z),
                                                   capi.ROW_F64, None, 4096, G.ptr(z), 1e-3, G.ptr(z), 10, None)
    assert rc == -1 and b"1024" in capi.kernel_lib().tsvm_last_error()
