"""The C-ABI libraries load without a GPU and export every symbol the headers under include/ declare;
compute calls fail loudly instead of falling back to a CPU path."""
import ctypes
import os
import re

import pytest

from thundersvm_amd import capi, model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tsvm_[a-z0-9_]+)\s*\(", text)))


def test_kernel_library_exports():
    lib = capi.kernel_lib()
    names = _declared("thundersvm_amd.h")
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(capi.SIGNATURES), set(names) ^ set(capi.SIGNATURES)
    assert lib.tsvm_version() >= 100


def test_model_library_exports():
    lib = model.host_lib()
    names = _declared("thundersvm_amd_model.h")
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), n


def test_scikit_interface_exports():
    """Every function the reference's Python package binds (thundersvm-scikit.cpp) is exported under its name."""
    lib = model.host_lib()
    text = open(os.path.join(ROOT, "include", "thundersvm_scikit.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b\*?([a-z_]+)\s*\(", text)) - {"defined"})
    assert len(names) == 26, names
    for n in names:
        assert hasattr(lib, n), n
    # no GPU needed for these
    lib.model_new.restype = ctypes.c_void_p
    m = lib.model_new(0)
    assert m and lib.model_new(9) is None
    n_model = (ctypes.c_int * 1)(7)
    lib.get_n_binary_models(ctypes.c_void_p(m), n_model)
    assert n_model[0] == 1
    assert lib.n_sv(ctypes.c_void_p(m)) == 0
    lib.model_free(ctypes.c_void_p(m))


def test_argument_checks_do_not_need_a_gpu():
    lib = capi.kernel_lib()
    rc = lib.tsvm_update_f(None, None, 4, None, 0, None, 8, 8, 1, None)
    assert rc == -1 and b"null pointer" in lib.tsvm_last_error()
    rc = lib.tsvm_get_rows_dense(8, 12, None, 4, 4, 8, 8, 12, None, 1, 8, 2, 0.5, 0.0, 3, 8, 0, None, 4, None)
    assert rc == -1 and b"multiples of 8" in lib.tsvm_last_error()
    assert lib.tsvm_select_workspace(1000) > 1000 * 10
    assert lib.tsvm_smo_solve_workspace(1024) >= 8 * 1024 * 1024


def test_no_cpu_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from thundersvm_amd import data as D
    w = D.workload_c1(0.05)
    with pytest.raises((capi.TsvmError, MemoryError)):
        model.Model(0).train(w["train"], model.make_param(**w["params"]))


def test_bounded_wait_for_the_local_solver():
    """The host's wait for the solver's report gives up with an error instead of spinning for ever (host only:
    the word is never written, no kernel is involved)."""
    import selftest_lib
    lib = selftest_lib.lib()
    assert lib.tsvm_selftest_solver_wait(300, 0) == 0, lib.tsvm_selftest_last_error()
    assert b"TSVM_SOLVER_TIMEOUT_MS" in lib.tsvm_selftest_last_error()
    assert lib.tsvm_selftest_solver_wait(60000, 1) == 0, lib.tsvm_selftest_last_error()
    assert b"without reporting" in lib.tsvm_selftest_last_error()


def test_row_cache_bookkeeping():
    """The kernel-row cache on scripted sequences (host only).  Ids come round in a cycle, as SMO's candidates roughly do.
    With a slot for every id each id misses once.  With fewer slots than ids, least-recently-used order would never hit
    (every row is evicted just before its turn comes again); rows that were computed leave at the tail instead, so a
    resident set survives and hits once per cycle.  After every iteration the hook checks that the working set's rows
    are pinned, own their slots and are off the eviction list."""
    import selftest_lib
    lib = selftest_lib.lib()
    ws, q = 64, 32
    # every id has a slot: each id misses exactly once
    n_ids, iters = 1000, 200
    lookups = ws + q * (iters - 1)
    assert lib.tsvm_selftest_row_cache(n_ids, 1000, ws, iters) == lookups - n_ids, lib.tsvm_selftest_last_error()
    # 1000 ids, 400 slots: a resident set of about 400 - ws rows hits in every later cycle
    hits = lib.tsvm_selftest_row_cache(n_ids, 400, ws, iters)
    assert hits >= 0, lib.tsvm_selftest_last_error()
    cycles = lookups // n_ids
    assert hits >= (cycles - 1) * 250, hits          # least-recently-used order: 0
    assert hits <= lookups - n_ids
    # the smallest cache the solver uses (four working sets) and a cycle barely longer than it
    assert lib.tsvm_selftest_row_cache(4 * ws + 8, 4 * ws, ws, 300) >= 0, lib.tsvm_selftest_last_error()
    assert lib.tsvm_selftest_row_cache(10, 400, ws, 10) == -1 and b"bad arguments" in lib.tsvm_selftest_last_error()
