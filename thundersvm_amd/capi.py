"""ctypes binding of the gfx950 kernel library's C ABI (include/thundersvm_amd.h).

Device buffers are passed as integer addresses; callers typically hold them as torch CUDA tensors
(`t.data_ptr()`), torch being used for device memory and streams only.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_LIB = os.path.join(_HERE, "libtsvm_hip.so")
HOST_LIB = os.path.join(_HERE, "libthundersvm.so")

LINEAR, POLY, RBF, SIGMOID, PRECOMPUTED = range(5)
C_SVC, NU_SVC, ONE_CLASS, EPSILON_SVR, NU_SVR = range(5)
ROW_F64, ROW_F32 = 0, 1

_p = C.c_void_p
_i64 = C.c_int64
_int = C.c_int
_dbl = C.c_double

SIGNATURES = {
    "tsvm_last_error": (C.c_char_p, []),
    "tsvm_version": (_int, []),
    "tsvm_csr_self_dot": (_int, [_p, _p, _i64, _p, _p]),
    "tsvm_dense_self_dot": (_int, [_p, _i64, _i64, _int, _p, _p]),
    "tsvm_kernel_diag": (_int, [_p, _i64, _int, _dbl, _dbl, _int, _p, _p]),
    "tsvm_csr_to_dense": (_int, [_p, _p, _p, _i64, _p, _i64, _p]),
    "tsvm_column_stats_dense": (_int, [_p, _i64, _i64, _int, _p, _p]),
    "tsvm_column_stats_csr": (_int, [_p, _p, _i64, _int, _p, _p]),
    "tsvm_indicator_masks": (_int, [_p, _i64, _i64, _int, _int, _p, _p, _p]),
    "tsvm_get_rows_dense_indicator": (_int, [_p, _i64, _p, _i64, _int, _p, _p, _p, _i64, _p, _int, _p, _p, _p, _int, _int, _dbl, _dbl,
                                             _int, _p, _int, _p, _i64, _p]),
    "tsvm_get_rows_dense": (_int, [_p, _i64, _p, _i64, _int, _p, _p, _i64, _p, _int, _p, _int, _dbl, _dbl, _int, _p, _int, _p, _i64, _p]),
    "tsvm_get_rows_dense_counted": (_int, [_p, _i64, _p, _i64, _int, _p, _p, _i64, _p, _int, _p, _p, _int, _dbl, _dbl, _int, _p, _int, _p, _i64, _p]),
    "tsvm_csr_stage_rows": (_int, [_p, _p, _p, _p, _int, _int, _p, _p]),
    "tsvm_csr_scatter_rows": (_int, [_p, _p, _p, _p, _int, _int, _p, _int, _int, _p]),
    "tsvm_get_rows_csr": (_int, [_p, _p, _p, _p, _i64, _p, _p, _int, _p, _int, _dbl, _dbl, _int, _p, _int, _p, _i64, _p]),
    "tsvm_get_rows_csr_staged": (_int, [_p, _p, _p, _p, _i64, _p, _p, _int, _int, _p, _int, _dbl, _dbl, _int, _p, _int, _p, _i64, _p]),
    "tsvm_csr_slice_widths": (_int, [_p, _i64, _p, _p]),
    "tsvm_csr_to_sliced": (_int, [_p, _p, _p, _i64, _p, _int, _p, _p, _int, _p]),
    "tsvm_get_rows_csr_sliced_lds": (C.c_size_t, [_int, _int, _int]),
    "tsvm_get_rows_csr_sliced": (_int, [_p, _p, _int, _p, _i64, _p, _p, _p, _p, _p, _int, _p, _int, _int, _int, _dbl, _dbl, _int,
                                        _p, _int, _p, _i64, _p]),
    "tsvm_fold_ids": (_int, [_p, _int, _int, _p, _p]),
    "tsvm_gather_rows_f64": (_int, [_p, _i64, _p, _i64, _p, _p]),
    "tsvm_csr_gather_rows": (_int, [_p, _p, _p, _p, _i64, _p, _p, _p, _p]),
    "tsvm_gather_f64": (_int, [_p, _p, _int, _p, _p]),
    "tsvm_update_f": (_int, [_p, _p, _int, _p, _int, _p, _i64, _i64, _int, _p]),
    "tsvm_smo_solve_workspace": (C.c_size_t, [_int]),
    "tsvm_c_smo_solve": (_int, [_p, _p, _p, _p, _p, _int, _dbl, _dbl, _p, _int, _p, _i64, _p, _dbl, _p, _int, _p, _p]),
    "tsvm_c_smo_solve_static_init": (_int, []),
    "tsvm_c_smo_solve_static": (_int, [_p, _p, _p, _p, _p, _int, _dbl, _dbl, _p, _int, _p, _i64, _p, _dbl, _p, _int, _p]),
    "tsvm_nu_smo_solve": (_int, [_p, _p, _p, _p, _p, _int, _dbl, _p, _int, _p, _i64, _p, _dbl, _p, _int, _p, _p]),
    "tsvm_smo_solve_block_ld": (_int, [_int]),
    "tsvm_smo_gather_block": (_int, [_p, _int, _p, _i64, _p, _int, _p, _int, _p]),
    "tsvm_row_slots_assign": (_int, [_p, _int, _p, _p, _p, _p, _p, _int, _p, _p, _p]),
    "tsvm_smo_gather_block_by_id": (_int, [_p, _int, _p, _i64, _p, _int, _p, _int, _p, _p]),
    "tsvm_c_smo_solve_block": (_int, [_p, _p, _p, _p, _p, _int, _dbl, _dbl, _p, _int, _p, _dbl, _p, _int, _p]),
    "tsvm_nu_smo_solve_block": (_int, [_p, _p, _p, _p, _p, _int, _dbl, _p, _int, _p, _dbl, _p, _int, _p]),
    "tsvm_c_smo_solve_block_on_xcd": (_int, [_p, _p, _p, _p, _p, _int, _dbl, _dbl, _p, _int, _p, _dbl, _p, _int, _p, _int, _int, _p]),
    "tsvm_nu_smo_solve_block_on_xcd": (_int, [_p, _p, _p, _p, _p, _int, _dbl, _p, _int, _p, _dbl, _p, _int, _p, _int, _int, _p]),
    "tsvm_select_workspace": (C.c_size_t, [_i64]),
    "tsvm_report_ids": (_int, [_p, _int, _int, _p, _int, _int, _p]),
    "tsvm_select_working_set": (_int, [_p, _p, _p, _i64, _dbl, _dbl, _p, _int, _p, _int, _int, _p, _p]),
    "tsvm_select_working_set_again": (_int, [_p, _p, _p, _i64, _dbl, _dbl, _p, _int, _p, _int, _int, _p, _p]),
    "tsvm_select_working_set_folded": (_int, [_p, _p, _p, _i64, _dbl, _dbl, _p, _int, _p, _int, _int, _p, _int, _int, _p, _p]),
    "tsvm_update_f_select": (_int, [_p, _p, _int, _p, _int, _p, _i64, _i64, _int, _p, _p, _dbl, _dbl, _p, _int, _p, _int, _int, _p, _p, _p]),
    "tsvm_sum_kernel_values": (_int, [_p, _int, _p, _p, _p, _p, _int, _i64, _p, _int, _i64, _p]),
    "tsvm_predict_nc_stride": (_int, [_int, _int, _int]),
    "tsvm_predict_dec_values_dense": (_int, [_p, _i64, _int, _p, _p, _p, _i64, _p, _p, _int, _p, _p, _int, _p, _i64, _i64, _p, _p,
                                             _int, _int, _dbl, _dbl, _int, _p, _p, _p]),
}

_LIB = None


class TsvmError(RuntimeError):
    pass


def kernel_lib():
    """Loads libtsvm_hip.so; raises if it has not been built (there is no CPU fallback)."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(KERNEL_LIB):
            raise TsvmError("%s is missing: run `python -m thundersvm_amd.build` (hipcc, gfx950)" % KERNEL_LIB)
        lib = C.CDLL(KERNEL_LIB, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _LIB = lib
    return _LIB


def check(rc):
    if rc != 0:
        msg = kernel_lib().tsvm_last_error().decode()
        if rc == 2:
            raise MemoryError(msg)
        raise TsvmError("tsvm call failed (%d): %s" % (rc, msg))


def call(name, *args):
    check(getattr(kernel_lib(), name)(*args))
