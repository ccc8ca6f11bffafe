"""Loads the test-only native library (tests/native/selftest.cpp, built by thundersvm_amd.build.build_selftests):
self-tests of host-layer pieces that no product entry point reaches."""
import ctypes
import os

from thundersvm_amd import model

_LIB = None


def lib():
    global _LIB
    if _LIB is None:
        model.host_lib()        # the product libraries it links against
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "libtsvm_selftest.so")
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: run `python -m thundersvm_amd.build`" % path)
        L = ctypes.CDLL(path)
        L.tsvm_selftest_last_error.restype = ctypes.c_char_p
        L.tsvm_selftest_row_cache.restype = ctypes.c_longlong
        L.tsvm_selftest_row_cache.argtypes = [ctypes.c_int] * 4
        L.tsvm_selftest_solver_wait.argtypes = [ctypes.c_int, ctypes.c_int]
        _LIB = L
    return _LIB
