"""Python face of the model-level C ABI (libthundersvm.so): train / predict / save / load.

Mirrors the reference's SvmModel surface (include/thundersvm/model/svmmodel.h:18-213) with float64
arrays; everything numeric happens in the C++ host layer and the gfx950 kernels.
"""
import ctypes as C
import os

import numpy as np

from . import capi
from .data import CsrData

_i64p = C.POINTER(C.c_int64)
_ip = C.POINTER(C.c_int)
_dp = C.POINTER(C.c_double)


class TsvmParam(C.Structure):
    _fields_ = [("svm_type", C.c_int), ("kernel_type", C.c_int), ("degree", C.c_int), ("max_iter", C.c_int),
                ("gamma", C.c_double), ("coef0", C.c_double), ("C", C.c_double), ("nu", C.c_double),
                ("p", C.c_double), ("epsilon", C.c_double), ("max_mem_size", C.c_int64), ("nr_weight", C.c_int),
                ("verbose", C.c_int), ("weight_label", _ip), ("weight", _dp), ("cache_bytes", C.c_int64), ("pair_lanes", C.c_int)]


def make_param(svm_type=0, kernel_type=2, degree=3, gamma=0.0, coef0=0.0, C=1.0, nu=0.5, p=0.1, epsilon=0.001,
               max_mem_size=8192 << 20, max_iter=-1, verbose=0, cache_bytes=-1, pair_lanes=0, weights=None):
    """Defaults of include/thundersvm/svmparam.h:14-29.  weights: {class label: factor on C} (the CLI's -wi)."""
    prm = TsvmParam()
    prm.svm_type, prm.kernel_type, prm.degree, prm.max_iter = svm_type, kernel_type, degree, max_iter
    prm.gamma, prm.coef0, prm.C, prm.nu, prm.p, prm.epsilon = gamma, coef0, C, nu, p, epsilon
    prm.max_mem_size, prm.nr_weight, prm.verbose = max_mem_size, 0, verbose
    prm.cache_bytes = cache_bytes
    prm.pair_lanes = pair_lanes
    if weights:
        prm._keep = (np.array(list(weights.keys()), dtype=np.int32), np.array(list(weights.values()), dtype=np.float64))
        prm.nr_weight = len(weights)
        prm.weight_label = prm._keep[0].ctypes.data_as(_ip)
        prm.weight = prm._keep[1].ctypes.data_as(_dp)
    return prm


_HOST = None


def host_lib():
    global _HOST
    if _HOST is None:
        capi.kernel_lib()
        if not os.path.exists(capi.HOST_LIB):
            raise capi.TsvmError("%s is missing: run `python -m thundersvm_amd.build`" % capi.HOST_LIB)
        L = C.CDLL(capi.HOST_LIB)
        L.tsvm_model_last_error.restype = C.c_char_p
        L.tsvm_model_new.restype = C.c_void_p
        L.tsvm_model_new.argtypes = [C.c_int]
        L.tsvm_model_free.argtypes = [C.c_void_p]
        L.tsvm_model_train_csr.argtypes = [C.c_void_p, C.c_int64, _i64p, _ip, _dp, _dp, C.POINTER(TsvmParam), C.c_int,
                                           C.c_int, C.c_int, C.c_int]
        L.tsvm_dataset_new_csr.restype = C.c_void_p
        L.tsvm_dataset_new_csr.argtypes = [C.c_int64, _i64p, _ip, _dp, _dp]
        L.tsvm_dataset_load.restype = C.c_void_p
        L.tsvm_dataset_load.argtypes = [C.c_char_p]
        L.tsvm_dataset_load_threads.restype = C.c_void_p
        L.tsvm_dataset_load_threads.argtypes = [C.c_char_p, C.c_int]
        L.tsvm_dataset_info.restype = C.c_int64
        L.tsvm_dataset_info.argtypes = [C.c_void_p, _i64p, _ip, _ip]
        L.tsvm_dataset_get_csr.restype = None
        L.tsvm_dataset_get_csr.argtypes = [C.c_void_p, _i64p, _ip, _dp, _dp]
        L.tsvm_rule_choose_dense.argtypes = [C.c_int64, C.c_int64, C.c_int64]
        L.tsvm_rule_indicator_run_start.argtypes = [_ip, C.c_int]
        L.tsvm_rule_indicator_run_pays.argtypes = [C.c_int, C.c_int, C.c_int]
        L.tsvm_dataset_free.argtypes = [C.c_void_p]
        L.tsvm_dataset_rows.restype = C.c_int64
        L.tsvm_dataset_rows.argtypes = [C.c_void_p]
        L.tsvm_dataset_to_device.argtypes = [C.c_void_p]
        L.tsvm_model_train.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(TsvmParam), C.c_int, C.c_int, C.c_int, C.c_int]
        L.tsvm_model_predict.argtypes = [C.c_void_p, C.c_void_p, C.c_int, _dp, _dp]
        L.tsvm_model_train_file.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(TsvmParam)]
        L.tsvm_model_info.argtypes = [C.c_void_p, _ip, _ip, _ip, _i64p]
        L.tsvm_model_get.argtypes = [C.c_void_p, _ip, _ip, _dp, _dp, _ip, _i64p, _ip, _dp]
        L.tsvm_model_stats.argtypes = [C.c_void_p, C.c_int, _i64p, _i64p, _dp, _dp]
        L.tsvm_model_binary_size.restype = C.c_int64
        L.tsvm_model_binary_size.argtypes = [C.c_void_p, C.c_int]
        L.tsvm_model_binary.argtypes = [C.c_void_p, C.c_int, _dp, _dp]
        L.tsvm_model_trace.argtypes = [C.c_void_p, _ip, C.POINTER(_dp), C.POINTER(_ip)]
        L.tsvm_model_predict_csr.argtypes = [C.c_void_p, C.c_int64, _i64p, _ip, _dp, C.c_int, _dp, _dp]
        L.tsvm_model_save.argtypes = [C.c_void_p, C.c_char_p]
        L.tsvm_model_load.argtypes = [C.c_void_p, C.c_char_p]
        _HOST = L
    return _HOST


def choose_dense(n, n_features, nnz):
    """KernelMatrix::choose_dense of the host layer: dense row-major rows (True) or CSR."""
    return bool(host_lib().tsvm_rule_choose_dense(n, n_features, nnz))


def indicator_run(column_stats, n_features, max_ones=None):
    """First column of the trailing run of 0/1 columns (the host layer's rule, from tsvm_column_stats_dense's counts);
    with max_ones also whether get_rows leaves the run to its epilogue."""
    counts = np.ascontiguousarray(column_stats, dtype=np.int32)
    first = host_lib().tsvm_rule_indicator_run_start(_p(counts, _ip), n_features)
    if max_ones is None:
        return first
    return first, bool(host_lib().tsvm_rule_indicator_run_pays(n_features, first, max_ones))


def _check(rc):
    if rc != 0:
        msg = host_lib().tsvm_model_last_error().decode()
        if rc == 2:
            raise MemoryError(msg or "device out of memory")
        raise capi.TsvmError(msg)


def _p(a, t):
    return None if a is None else a.ctypes.data_as(t)


class Dataset:
    """Rows held by the host layer's DataSet (converted once, reusable across train / predict calls)."""

    def __init__(self, data=None, path=None, threads=0):
        L = host_lib()
        if path is not None:
            self.h = C.c_void_p(L.tsvm_dataset_load_threads(path.encode(), threads))
        else:
            y = None if data.y is None else np.ascontiguousarray(data.y, dtype=np.float64)
            self.h = C.c_void_p(L.tsvm_dataset_new_csr(data.n, _p(data.ptr, _i64p), _p(data.col, _ip), _p(data.val, _dp),
                                                       _p(y, _dp)))
        if not self.h:
            raise capi.TsvmError(L.tsvm_model_last_error().decode())
        self.n = L.tsvm_dataset_rows(self.h)

    def csr(self):
        """The rows as the DataSet holds them: CsrData with the stored feature ids, plus (n_features, zero_based)."""
        from .data import CsrData
        L = host_lib()
        nf, zb, hl = C.c_int64(), C.c_int(), C.c_int()
        nnz = L.tsvm_dataset_info(self.h, C.byref(nf), C.byref(zb), C.byref(hl))
        ptr = np.zeros(self.n + 1, dtype=np.int64)
        col = np.zeros(nnz, dtype=np.int32)
        val = np.zeros(nnz)
        y = np.zeros(self.n)
        L.tsvm_dataset_get_csr(self.h, _p(ptr, _i64p), _p(col, _ip), _p(val, _dp), _p(y, _dp))
        return CsrData(ptr, col, val, y if hl.value else None), nf.value, bool(zb.value)

    def to_device(self):
        """Uploads the rows to HBM now; training calls on this Dataset then start from device-resident data."""
        if host_lib().tsvm_dataset_to_device(self.h) != 0:
            raise capi.TsvmError(host_lib().tsvm_model_last_error().decode())
        return self

    def __del__(self):
        if getattr(self, "h", None):
            host_lib().tsvm_dataset_free(self.h)
            self.h = None


class Model:
    def __init__(self, svm_type=0):
        self.svm_type = svm_type
        self.h = C.c_void_p(host_lib().tsvm_model_new(svm_type))
        if not self.h:
            raise capi.TsvmError(host_lib().tsvm_model_last_error().decode())

    def __del__(self):
        if getattr(self, "h", None):
            host_lib().tsvm_model_free(self.h)
            self.h = None

    def train(self, data, param, ws_override=0, keep_binary=False, trace_cap=0, profile=False):
        if isinstance(data, Dataset):
            _check(host_lib().tsvm_model_train(self.h, data.h, C.byref(param), ws_override, int(keep_binary), trace_cap,
                                               int(profile)))
            self._fetch()
            return self
        y = data.y if data.y is not None else np.zeros(data.n)
        _check(host_lib().tsvm_model_train_csr(self.h, data.n, _p(data.ptr, _i64p), _p(data.col, _ip), _p(data.val, _dp),
                                               _p(np.ascontiguousarray(y, dtype=np.float64), _dp), C.byref(param),
                                               ws_override, int(keep_binary), trace_cap, int(profile)))
        self._fetch()
        return self

    def train_file(self, path, param):
        _check(host_lib().tsvm_model_train_file(self.h, path.encode(), C.byref(param)))
        self._fetch()
        return self

    def _fetch(self):
        L = host_lib()
        nc, nb, tsv, nnz = C.c_int(), C.c_int(), C.c_int(), C.c_int64()
        _check(L.tsvm_model_info(self.h, C.byref(nc), C.byref(nb), C.byref(tsv), C.byref(nnz)))
        self.n_classes, self.n_binary, self.total_sv = nc.value, nb.value, tsv.value
        cls = self.svm_type in (0, 1)
        self.label = np.zeros(self.n_classes, dtype=np.int32)
        self.n_sv = np.zeros(self.n_classes, dtype=np.int32)
        self.rho = np.zeros(self.n_binary)
        self.coef = np.zeros((self.n_classes - 1) * self.total_sv if cls else self.total_sv)
        self.sv_indices = np.zeros(self.total_sv, dtype=np.int32)
        _check(L.tsvm_model_get(self.h, _p(self.label, _ip), _p(self.n_sv, _ip), _p(self.rho, _dp), _p(self.coef, _dp),
                                _p(self.sv_indices, _ip), None, None, None))
        self._sv_nnz = nnz.value
        self._sv = None   # the support vectors' CSR copy is made when first asked for (sv_ptr / sv_col / sv_val)

    def _support_vectors(self):
        if self._sv is None:
            sv_ptr = np.zeros(self.total_sv + 1, dtype=np.int64)
            sv_col = np.zeros(self._sv_nnz, dtype=np.int32)
            sv_val = np.zeros(self._sv_nnz)
            _check(host_lib().tsvm_model_get(self.h, None, None, None, None, None, _p(sv_ptr, _i64p), _p(sv_col, _ip),
                                             _p(sv_val, _dp)))
            self._sv = (sv_ptr, sv_col, sv_val)
        return self._sv

    @property
    def sv_ptr(self):
        return self._support_vectors()[0]

    @property
    def sv_col(self):
        return self._support_vectors()[1]

    @property
    def sv_val(self):
        return self._support_vectors()[2]

    def stats(self, k=0):
        ni, li, obj = C.c_int64(), C.c_int64(), C.c_double()
        ms = np.zeros(16)
        _check(host_lib().tsvm_model_stats(self.h, k, C.byref(ni), C.byref(li), C.byref(obj), _p(ms, _dp)))
        return dict(n_iter=ni.value, local_iter=li.value, obj=obj.value, ms_select=ms[0], ms_get_rows=ms[1],
                    ms_local=ms[2], ms_update_f=ms[3], cache_lookups=int(ms[4]), cache_hits=int(ms[5]), cache_rows=int(ms[6]),
                    cache_disabled=bool(ms[7]), ms_wall=ms[8], ms_setup=ms[9], ws_size=int(ms[10]),
                    rows_computed=int(ms[11]), update_rows=int(ms[12]), solver_xcd=int(ms[13]),
                    ms_start=ms[14], ms_end=ms[15])

    def binary(self, k):
        n = host_lib().tsvm_model_binary_size(self.h, k)
        a, f = np.zeros(n), np.zeros(n)
        _check(host_lib().tsvm_model_binary(self.h, k, _p(a, _dp), _p(f, _dp)))
        return a, f

    def trace(self):
        ws_size = C.c_int()
        d, w = _dp(), _ip()
        n = host_lib().tsvm_model_trace(self.h, C.byref(ws_size), C.byref(d), C.byref(w))
        if n == 0:
            return np.zeros((0, 2)), np.zeros((0, 0), dtype=np.int32)
        return (np.ctypeslib.as_array(d, shape=(n, 2)).copy(),
                np.ctypeslib.as_array(w, shape=(n, ws_size.value)).copy())

    def predict(self, data, batch_size=-1):
        """Returns (labels / values, decision values [n, n_binary])."""
        dec = np.zeros((data.n, self.n_binary))
        lab = np.zeros(data.n)
        if isinstance(data, Dataset):
            _check(host_lib().tsvm_model_predict(self.h, data.h, batch_size, _p(dec, _dp), _p(lab, _dp)))
            return lab, dec
        _check(host_lib().tsvm_model_predict_csr(self.h, data.n, _p(data.ptr, _i64p), _p(data.col, _ip),
                                                 _p(data.val, _dp), batch_size, _p(dec, _dp), _p(lab, _dp)))
        return lab, dec

    def cross_validation(self, dataset, prm, n_fold):
        """SvmModel::cross_validation on a Dataset: the out-of-fold prediction of every instance."""
        L = host_lib()
        L.tsvm_model_cross_validation.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(TsvmParam), C.c_int, _dp]
        out = np.zeros(dataset.n)
        _check(L.tsvm_model_cross_validation(self.h, dataset.h, C.byref(prm), n_fold, _p(out, _dp)))
        return out

    def save(self, path):
        _check(host_lib().tsvm_model_save(self.h, path.encode()))

    def load(self, path):
        _check(host_lib().tsvm_model_load(self.h, path.encode()))
        self._fetch()
        return self
