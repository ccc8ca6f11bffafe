"""Helpers for the GPU parity tests: device buffers through torch, calls through the C ABI."""
import numpy as np
import torch

from thundersvm_amd import capi


def dev(a, dtype=None):
    a = np.ascontiguousarray(a, dtype=dtype)
    return torch.from_numpy(a).cuda()


def ptr(t):
    return None if t is None else t.data_ptr()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def stream():
    return torch.cuda.current_stream().cuda_stream or None


def round_up(v, m):
    return (v + m - 1) // m * m


def dense_padded(data, n_cols=None):
    """CsrData -> float64 [n, ld] with ld = n_features+1 rounded up to 8 (column c = feature id c)."""
    nf = (n_cols if n_cols is not None else data.n_features + 1)
    ld = round_up(max(nf, 1), 8)
    return data.to_dense(ld), nf, ld


def get_rows_dense(x_d, ld, n, d, sd_x, a_d, lda, a_idx, m, sd_a, kernel_type, gamma=0.0, coef0=0.0, degree=3,
                   out_slots=None, out_rows=None, x_idx=None, row_type=capi.ROW_F64):
    """Rows come back as float64 (row_type F64) or float32 (F32) torch tensors."""
    dt = torch.float32 if row_type == capi.ROW_F32 else torch.float64
    out = torch.empty((out_rows or m, n), dtype=dt, device="cuda")
    capi.call("tsvm_get_rows_dense", ptr(x_d), ld, ptr(x_idx), n, d, ptr(sd_x), ptr(a_d), lda, ptr(a_idx), m, ptr(sd_a),
              kernel_type, gamma, coef0, degree, ptr(out), row_type, ptr(out_slots), n, stream())
    return out


def float_ulp_diff(a, b):
    """Distance in float32 ulps between two float32-exact float64 arrays."""
    ia = np.asarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    ib = np.asarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7fffffff), ia)
    ib = np.where(ib < 0, -(ib & 0x7fffffff), ib)
    return np.abs(ia - ib)
