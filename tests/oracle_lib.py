"""ctypes binding of the CPU oracle (oracle/liboracle.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
_LIB = None

C_SVC, NU_SVC, ONE_CLASS, EPSILON_SVR, NU_SVR = range(5)
LINEAR, POLY, RBF, SIGMOID, PRECOMPUTED = range(5)


class OrcParam(C.Structure):
    _fields_ = [("svm_type", C.c_int), ("kernel_type", C.c_int), ("degree", C.c_int), ("expf_mode", C.c_int),
                ("gamma", C.c_double), ("coef0", C.c_double), ("C", C.c_double), ("nu", C.c_double),
                ("p", C.c_double), ("epsilon", C.c_double), ("max_mem_size", C.c_longlong), ("max_iter", C.c_int),
                ("nr_weight", C.c_int), ("weight_label", C.POINTER(C.c_int)), ("weight", C.POINTER(C.c_double))]


def make_param(svm_type=C_SVC, kernel_type=RBF, degree=3, gamma=0.0, coef0=0.0, C_=1.0, nu=0.5, p=0.1,
               epsilon=0.001, max_mem_size=8192 << 20, max_iter=-1, expf_mode=1, weights=None):
    """Defaults follow include/thundersvm/svmparam.h:14-29 (p and epsilon are float literals there).
    weights: {class label: factor on C}."""
    prm = OrcParam()
    prm.svm_type, prm.kernel_type, prm.degree, prm.expf_mode = svm_type, kernel_type, degree, expf_mode
    prm.gamma, prm.coef0, prm.C, prm.nu = gamma, coef0, C_, nu
    prm.p, prm.epsilon = p, epsilon
    prm.max_mem_size, prm.max_iter, prm.nr_weight = max_mem_size, max_iter, 0
    if weights:
        prm._keep = (np.array(list(weights.keys()), dtype=np.int32), np.array(list(weights.values()), dtype=np.float64))
        prm.nr_weight = len(weights)
        prm.weight_label = prm._keep[0].ctypes.data_as(C.POINTER(C.c_int))
        prm.weight = prm._keep[1].ctypes.data_as(C.POINTER(C.c_double))
    return prm


def _ptr(a, t):
    return a.ctypes.data_as(C.POINTER(t)) if a is not None else None


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(ORACLE_DIR, "liboracle.so")
        if not os.path.exists(so):
            subprocess.check_call(["make", "-C", ORACLE_DIR])
        L = C.CDLL(so)
        L.orc_expf_det.restype = C.c_float
        L.orc_expf_det.argtypes = [C.c_float]
        L.orc_expf_libm.restype = C.c_float
        L.orc_expf_libm.argtypes = [C.c_float]
        L.orc_expf_count_mismatch.restype = C.c_longlong
        L.orc_expf_count_mismatch.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32)]
        L.orc_powf_det.restype = C.c_float
        L.orc_powf_det.argtypes = [C.c_float, C.c_float]
        L.orc_tanhf_det.restype = C.c_float
        L.orc_tanhf_det.argtypes = [C.c_float]
        L.orc_expm1f_det.restype = C.c_float
        L.orc_expm1f_det.argtypes = [C.c_float]
        L.orc_powf_count_mismatch.restype = C.c_longlong
        L.orc_powf_count_mismatch.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_float, C.POINTER(C.c_uint32)]
        L.orc_tanhf_count_mismatch.restype = C.c_longlong
        L.orc_tanhf_count_mismatch.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32)]
        L.orc_km_create.restype = C.c_void_p
        L.orc_train.restype = C.c_void_p
        L.orc_calculate_rho.restype = C.c_double
        L.orc_calculate_obj.restype = C.c_double
        L.orc_model_sv_nnz.restype = C.c_longlong
        L.orc_model_binary_size.restype = C.c_longlong
        for name in ("orc_is_I_up", "orc_is_I_low", "orc_is_free"):
            getattr(L, name).argtypes = [C.c_double] * 4
        L.orc_max2power.argtypes = [C.c_longlong]
        L.orc_working_set_size.argtypes = [C.c_longlong] * 4
        _LIB = L
    return _LIB


def csr_arrays(ptr, col, val):
    return (np.ascontiguousarray(ptr, dtype=np.int64), np.ascontiguousarray(col, dtype=np.int32),
            np.ascontiguousarray(val, dtype=np.float64))


class KernelMatrix:
    """Oracle KernelMatrix over CSR rows (kernelmatrix.cpp:183-316)."""

    def __init__(self, ptr, col, val, param):
        self.ptr, self.col, self.val = csr_arrays(ptr, col, val)
        self.n = len(self.ptr) - 1
        self.param = param
        self.h = C.c_void_p(lib().orc_km_create(C.c_int(self.n), _ptr(self.ptr, C.c_longlong), _ptr(self.col, C.c_int),
                                                _ptr(self.val, C.c_double), C.byref(param)))

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_km_free(self.h)
            self.h = None

    @property
    def n_features(self):
        return lib().orc_km_n_features(self.h)

    def self_dot(self):
        out = np.empty(self.n)
        lib().orc_km_self_dot(self.h, _ptr(out, C.c_double))
        return out

    def diag(self):
        out = np.empty(self.n)
        lib().orc_km_diag(self.h, _ptr(out, C.c_double))
        return out

    def get_rows(self, idx):
        idx = np.ascontiguousarray(idx, dtype=np.int32)
        out = np.empty((len(idx), self.n))
        lib().orc_km_get_rows(self.h, _ptr(idx, C.c_int), C.c_int(len(idx)), _ptr(out, C.c_double))
        return out

    def get_rows_instances(self, bptr, bcol, bval):
        bptr, bcol, bval = csr_arrays(bptr, bcol, bval)
        m = len(bptr) - 1
        out = np.empty((m, self.n))
        lib().orc_km_get_rows_instances(self.h, C.c_int(m), _ptr(bptr, C.c_longlong), _ptr(bcol, C.c_int),
                                        _ptr(bval, C.c_double), _ptr(out, C.c_double))
        return out


def sort_f(f):
    f = np.ascontiguousarray(f, dtype=np.float64)
    idx = np.arange(len(f), dtype=np.int32)
    lib().orc_sort_f(_ptr(f, C.c_double), _ptr(idx, C.c_int), C.c_int(len(f)))
    return idx


def select_working_set(f, y, alpha, Cp, Cn, marked, n_select, nu=False):
    f = np.ascontiguousarray(f, dtype=np.float64)
    y = np.ascontiguousarray(y, dtype=np.int32)
    alpha = np.ascontiguousarray(alpha, dtype=np.float64)
    marked = np.ascontiguousarray(marked, dtype=np.int32)
    out = np.full(n_select, -1, dtype=np.int32)
    lib().orc_select_working_set(_ptr(f, C.c_double), _ptr(y, C.c_int), _ptr(alpha, C.c_double), C.c_int(len(f)),
                                 C.c_double(Cp), C.c_double(Cn), _ptr(marked, C.c_int), C.c_int(len(marked)),
                                 _ptr(out, C.c_int), C.c_int(n_select), C.c_int(int(nu)))
    return out


def c_smo_solve(y, f, alpha, ws, Cp, Cn, k_rows, diag, row_len, eps, max_iter):
    """Returns (f_unchanged, alpha_new, alpha_diff, diff); f is not written by c_smo_solve."""
    y = np.ascontiguousarray(y, dtype=np.int32)
    f = np.array(f, dtype=np.float64)
    alpha = np.array(alpha, dtype=np.float64)
    ws = np.ascontiguousarray(ws, dtype=np.int32)
    k_rows = np.ascontiguousarray(k_rows, dtype=np.float64)
    diag = np.ascontiguousarray(diag, dtype=np.float64)
    alpha_diff = np.zeros(len(ws))
    diff = np.zeros(2)
    lib().orc_c_smo_solve(_ptr(y, C.c_int), _ptr(f, C.c_double), _ptr(alpha, C.c_double), _ptr(alpha_diff, C.c_double),
                          _ptr(ws, C.c_int), C.c_int(len(ws)), C.c_double(Cp), C.c_double(Cn),
                          _ptr(k_rows, C.c_double), _ptr(diag, C.c_double), C.c_longlong(row_len), C.c_double(eps),
                          _ptr(diff, C.c_double), C.c_int(max_iter))
    return alpha, alpha_diff, diff


def nu_smo_solve(y, f, alpha, ws, Cc, k_rows, diag, row_len, eps, max_iter):
    y = np.ascontiguousarray(y, dtype=np.int32)
    f = np.array(f, dtype=np.float64)
    alpha = np.array(alpha, dtype=np.float64)
    ws = np.ascontiguousarray(ws, dtype=np.int32)
    k_rows = np.ascontiguousarray(k_rows, dtype=np.float64)
    diag = np.ascontiguousarray(diag, dtype=np.float64)
    alpha_diff = np.zeros(len(ws))
    diff = np.zeros(2)
    lib().orc_nu_smo_solve(_ptr(y, C.c_int), _ptr(f, C.c_double), _ptr(alpha, C.c_double), _ptr(alpha_diff, C.c_double),
                           _ptr(ws, C.c_int), C.c_int(len(ws)), C.c_double(Cc), _ptr(k_rows, C.c_double),
                           _ptr(diag, C.c_double), C.c_longlong(row_len), C.c_double(eps), _ptr(diff, C.c_double),
                           C.c_int(max_iter))
    return alpha, alpha_diff, diff


def update_f(f, alpha_diff, k_rows, n):
    f = np.array(f, dtype=np.float64)
    alpha_diff = np.ascontiguousarray(alpha_diff, dtype=np.float64)
    k_rows = np.ascontiguousarray(k_rows, dtype=np.float64)
    lib().orc_update_f(_ptr(f, C.c_double), _ptr(alpha_diff, C.c_double), C.c_int(len(alpha_diff)),
                       _ptr(k_rows, C.c_double), C.c_longlong(n))
    return f


def sum_kernel_values(coef, total_sv, sv_start, sv_count, rho, k_mat, n_classes, n_instances):
    coef = np.ascontiguousarray(coef, dtype=np.float64)
    sv_start = np.ascontiguousarray(sv_start, dtype=np.int32)
    sv_count = np.ascontiguousarray(sv_count, dtype=np.int32)
    rho = np.ascontiguousarray(rho, dtype=np.float64)
    k_mat = np.ascontiguousarray(k_mat, dtype=np.float64)
    nb = n_classes * (n_classes - 1) // 2
    dec = np.zeros((n_instances, nb))
    lib().orc_sum_kernel_values(_ptr(coef, C.c_double), C.c_int(total_sv), _ptr(sv_start, C.c_int),
                                _ptr(sv_count, C.c_int), _ptr(rho, C.c_double), _ptr(k_mat, C.c_double),
                                _ptr(dec, C.c_double), C.c_int(n_classes), C.c_int(n_instances))
    return dec


def smo_solve(km, y, alpha, f, eps, Cp, Cn, ws_size, out_max_iter=-1, nu=False, for_svr=False, trace_cap=0):
    """CSMOSolver::solve / NuSMOSolver::solve on an oracle KernelMatrix.  Returns a dict."""
    y = np.ascontiguousarray(y, dtype=np.int32)
    alpha = np.array(alpha, dtype=np.float64)
    f = np.array(f, dtype=np.float64)
    rho = C.c_double(0)
    obj = C.c_double(0)
    stats = np.zeros(2, dtype=np.int64)
    tdiff = np.zeros((max(trace_cap, 1), 2))
    tws = np.full((max(trace_cap, 1), ws_size), -1, dtype=np.int32)
    lib().orc_smo_solve(km.h, _ptr(y, C.c_int), _ptr(alpha, C.c_double), C.byref(rho), _ptr(f, C.c_double),
                        C.c_double(eps), C.c_double(Cp), C.c_double(Cn), C.c_int(ws_size), C.c_int(out_max_iter),
                        C.c_int(int(nu)), C.c_int(int(for_svr)), C.c_int(trace_cap),
                        _ptr(tdiff, C.c_double) if trace_cap else None, _ptr(tws, C.c_int) if trace_cap else None,
                        _ptr(stats, C.c_longlong), C.byref(obj))
    return dict(alpha=alpha, f=f, rho=rho.value, obj=obj.value, n_iter=int(stats[0]), local_iter=int(stats[1]),
                trace_diff=tdiff[:min(trace_cap, int(stats[0]))], trace_ws=tws[:min(trace_cap, int(stats[0]))])


class Model:
    """Oracle model: SVC / NuSVC / OneClassSVC / SVR / NuSVR train + predict."""

    def __init__(self, ptr, col, val, y, param, ws_override=0, want_trace=False):
        ptr, col, val = csr_arrays(ptr, col, val)
        y = np.ascontiguousarray(y, dtype=np.float64)
        n = len(ptr) - 1
        self.param = param
        L = lib()
        self.h = C.c_void_p(L.orc_train(C.c_int(n), _ptr(ptr, C.c_longlong), _ptr(col, C.c_int), _ptr(val, C.c_double),
                                        _ptr(y, C.c_double), C.byref(param), C.c_int(ws_override),
                                        C.c_int(int(want_trace))))
        self.n_classes = L.orc_model_n_classes(self.h)
        self.n_binary = L.orc_model_n_binary(self.h)
        self.total_sv = L.orc_model_total_sv(self.h)
        nnz = L.orc_model_sv_nnz(self.h)
        self.label = np.zeros(self.n_classes, dtype=np.int32)
        self.n_sv = np.zeros(self.n_classes, dtype=np.int32)
        self.rho = np.zeros(self.n_binary)
        ncoef = (self.n_classes - 1) * self.total_sv if param.svm_type in (C_SVC, NU_SVC) else self.total_sv
        self.coef = np.zeros(ncoef)
        self.sv_indices = np.zeros(self.total_sv, dtype=np.int32)
        self.sv_ptr = np.zeros(self.total_sv + 1, dtype=np.int64)
        self.sv_col = np.zeros(nnz, dtype=np.int32)
        self.sv_val = np.zeros(nnz)
        self.n_iter = np.zeros(self.n_binary, dtype=np.int64)
        self.local_iter = np.zeros(self.n_binary, dtype=np.int64)
        self.obj = np.zeros(self.n_binary)
        L.orc_model_get(self.h, _ptr(self.label, C.c_int), _ptr(self.n_sv, C.c_int), _ptr(self.rho, C.c_double),
                        _ptr(self.coef, C.c_double), _ptr(self.sv_indices, C.c_int), _ptr(self.sv_ptr, C.c_longlong),
                        _ptr(self.sv_col, C.c_int), _ptr(self.sv_val, C.c_double), _ptr(self.n_iter, C.c_longlong),
                        _ptr(self.local_iter, C.c_longlong), _ptr(self.obj, C.c_double))

    def __del__(self):
        if getattr(self, "h", None):
            lib().orc_model_free(self.h)
            self.h = None

    def binary(self, k):
        n = lib().orc_model_binary_size(self.h, C.c_int(k))
        a = np.zeros(n)
        f = np.zeros(n)
        lib().orc_model_binary_get(self.h, C.c_int(k), _ptr(a, C.c_double), _ptr(f, C.c_double))
        return a, f

    def trace(self):
        ws_size = C.c_int(0)
        d = C.POINTER(C.c_double)()
        w = C.POINTER(C.c_int)()
        n = lib().orc_model_trace(self.h, C.byref(ws_size), C.byref(d), C.byref(w))
        diff = np.ctypeslib.as_array(d, shape=(n, 2)).copy() if n else np.zeros((0, 2))
        ws = np.ctypeslib.as_array(w, shape=(n, ws_size.value)).copy() if n else np.zeros((0, 0), dtype=np.int32)
        return diff, ws

    def predict_dec_values(self, bptr, bcol, bval, batch_size=10000):
        bptr, bcol, bval = csr_arrays(bptr, bcol, bval)
        m = len(bptr) - 1
        dec = np.zeros((m, self.n_binary))
        lib().orc_predict_dec_values(self.h, C.c_int(m), _ptr(bptr, C.c_longlong), _ptr(bcol, C.c_int),
                                     _ptr(bval, C.c_double), _ptr(dec, C.c_double), C.c_int(batch_size))
        return dec

    def predict(self, bptr, bcol, bval, batch_size=10000):
        dec = self.predict_dec_values(bptr, bcol, bval, batch_size)
        out = np.zeros(len(dec))
        lib().orc_predict_label(self.h, _ptr(dec, C.c_double), C.c_int(len(dec)), _ptr(out, C.c_double))
        return out, dec


# ---------------------------------------------------------------------------------------------
# Probability estimates (svc.cpp:197-491)
# ---------------------------------------------------------------------------------------------
def sigmoid_predict(dec, A, B):
    L = lib()
    L.orc_sigmoid_predict.restype = C.c_double
    return L.orc_sigmoid_predict(C.c_double(dec), C.c_double(A), C.c_double(B))


def sigmoid_train(dec, labels):
    dec = np.ascontiguousarray(dec, dtype=np.float64)
    labels = np.ascontiguousarray(labels, dtype=np.int32)
    a, b = C.c_double(), C.c_double()
    lib().orc_sigmoid_train(_ptr(dec, C.c_double), C.c_int(len(dec)), _ptr(labels, C.c_int), C.byref(a), C.byref(b))
    return a.value, b.value


def multiclass_probability(r):
    r = np.ascontiguousarray(r, dtype=np.float64)
    p = np.zeros(len(r))
    lib().orc_multiclass_probability(_ptr(r, C.c_double), C.c_int(len(r)), _ptr(p, C.c_double))
    return p


def _rows(ptr, col, val, idx):
    idx = np.asarray(idx, dtype=np.int64)
    lens = ptr[idx + 1] - ptr[idx]
    out_ptr = np.zeros(len(idx) + 1, dtype=np.int64)
    np.cumsum(lens, out=out_ptr[1:])
    take = np.repeat(ptr[idx] - out_ptr[:-1], lens) + np.arange(out_ptr[-1])
    return out_ptr, col[take], val[take]


def probability_train(ptr, col, val, y, param):
    """SVC::probability_train (svc.cpp:432-491): decision values of every instance from a 5-fold cross-validation
    (folds cut class by class in grouped order, class order = first appearance, dataset.cpp:199-214), then
    sigmoidTrain per class pair.  Returns (probA, probB)."""
    ptr, col, val = csr_arrays(ptr, col, val)
    y = np.asarray(y, dtype=np.float64)
    labels = list(dict.fromkeys(y.astype(np.int64).tolist()))
    groups = [np.flatnonzero(y.astype(np.int64) == c) for c in labels]
    k_cls = len(labels)
    n_binary = k_cls * (k_cls - 1) // 2
    dec_all = np.zeros((len(y), n_binary))
    n_fold = 5
    for fold in range(n_fold):
        train_idx, test_idx = [], []
        for ids in groups:
            per = len(ids) // n_fold
            b = per * fold
            e = len(ids) if fold == n_fold - 1 else min(len(ids), b + per)
            test_idx.extend(ids[b:e])
            train_idx.extend(np.concatenate([ids[:b], ids[e:]]))
        tp, tc, tv = _rows(ptr, col, val, train_idx)
        m = Model(tp, tc, tv, y[train_idx], param)
        sp_, sc, sv = _rows(ptr, col, val, test_idx)
        dec_all[test_idx] = m.predict_dec_values(sp_, sc, sv, 1000)
    prob_a, prob_b = np.zeros(n_binary), np.zeros(n_binary)
    k = 0
    for i in range(k_cls):
        for j in range(i + 1, k_cls):
            ids = np.concatenate([groups[i], groups[j]])
            lab = np.concatenate([np.ones(len(groups[i]), dtype=np.int32), -np.ones(len(groups[j]), dtype=np.int32)])
            prob_a[k], prob_b[k] = sigmoid_train(dec_all[ids, k], lab)
            k += 1
    return prob_a, prob_b


def predict_probability(dec, prob_a, prob_b, n_classes):
    """The probability branch of SVC::predict_label (svc.cpp:289-314): per row the coupled class probabilities."""
    out = np.zeros((len(dec), n_classes))
    for row in range(len(dec)):
        r = np.zeros((n_classes, n_classes))
        k = 0
        for i in range(n_classes):
            for j in range(i + 1, n_classes):
                r[i, j] = min(max(sigmoid_predict(dec[row, k], prob_a[k], prob_b[k]), 1e-7), 1 - 1e-7)
                r[j, i] = 1 - r[i, j]
                k += 1
        out[row] = multiclass_probability(r)
    return out
