"""Pins the restated expf (oracle orc_expf_det, also what the HIP epilogue computes) against libm's
expf on this host and against correctly rounded exp."""
import ctypes as C
import struct

import numpy as np

import oracle_lib as O


def _bits(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def test_matches_libm_on_rbf_range():
    """Every 97th float in [-104, -0] (11.5 million arguments): at most a handful differ from libm."""
    bad = C.c_uint32(0)
    n_bad = O.lib().orc_expf_count_mismatch(_bits(-0.0), _bits(-104.0), 97, C.byref(bad))
    total = (_bits(-104.0) - _bits(-0.0)) // 97 + 1
    assert n_bad <= total * 1e-6, (n_bad, hex(bad.value))


def test_correct_rounding_sample():
    rng = np.random.default_rng(11)
    x = np.concatenate([-rng.random(20000) * 100, -rng.random(20000), [0.0, -0.0, -103.9, -104.5, -1e-30, 1e-10]])
    x32 = x.astype(np.float32)
    f = O.lib().orc_expf_det
    got = np.array([f(float(v)) for v in x32], dtype=np.float32)
    want = np.exp(x32.astype(np.float64)).astype(np.float32)   # double exp rounded once more to float
    ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
    assert ulp.max() <= 1
    assert (ulp > 0).mean() < 1e-3


def test_special_values():
    f = O.lib().orc_expf_det
    assert f(0.0) == 1.0 and f(-0.0) == 1.0
    assert f(float("-inf")) == 0.0 and f(-200.0) == 0.0
    assert f(float("inf")) == float("inf") and f(89.0) == float("inf")
    assert np.isnan(f(float("nan")))
    assert f(1.0) == np.float32(np.e)
