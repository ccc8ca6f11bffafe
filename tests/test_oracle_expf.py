"""Pins the restated expf, powf and tanhf (oracle orc_expf_det / orc_powf_det / orc_tanhf_det, also what the HIP epilogues
compute) against libm's on this host and against correctly rounded values."""
import ctypes as C
import struct

import math

import numpy as np
import pytest

import oracle_lib as O


def _bits(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def test_matches_libm_on_rbf_range():
    """Every 97th float in [-104, -0] (11.5 million arguments) and every 1009th float pattern of all: libm's bits (the
    sweep of all 2^32 arguments, run once, found no difference; NaNs are compared as NaNs)."""
    bad = C.c_uint32(0)
    n_bad = O.lib().orc_expf_count_mismatch(_bits(-0.0), _bits(-104.0), 97, C.byref(bad))
    assert n_bad == 0, (n_bad, hex(bad.value))
    n_bad = O.lib().orc_expf_count_mismatch(0, 0xFFFFFFFF, 1009, C.byref(bad))
    assert n_bad == 0, (n_bad, hex(bad.value))
    # the two arguments on which the routine with a separately rounded product x * 32/ln2 differs from libm
    for x in (32.564632415771484, -63.09946060180664):
        assert O.lib().orc_expf_det(x) == O.lib().orc_expf_libm(x)


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


@pytest.mark.parametrize("y", [2.0, 3.0, 5.0, 8.0, 0.0, 1.0, -2.0, 2.5])
def test_powf_matches_libm(y):
    """Every 1009th float pattern (4.3 million arguments, all signs, subnormals, infinities, NaNs) for a given exponent:
    the restated powf gives libm's bits.  (The full sweep of all 2^32 arguments, run once for each of the exponents
    0.5, 1 ... 10, 17, -1, -2, 0 and 2.5, found no difference either.)"""
    bad = C.c_uint32(0)
    n_bad = O.lib().orc_powf_count_mismatch(0, 0xFFFFFFFF, 1009, y, C.byref(bad))
    assert n_bad == 0, (n_bad, hex(bad.value))


def test_powf_special_values():
    f = O.lib().orc_powf_det
    assert f(2.0, 3.0) == 8.0 and f(-2.0, 3.0) == -8.0 and f(-2.0, 2.0) == 4.0
    assert f(0.0, 3.0) == 0.0 and f(0.0, 0.0) == 1.0 and f(float("nan"), 0.0) == 1.0
    assert math.copysign(1.0, f(-0.0, 3.0)) == -1.0 and math.copysign(1.0, f(-0.0, 2.0)) == 1.0
    assert f(1e30, 3.0) == float("inf") and f(-1e30, 3.0) == float("-inf") and f(1e-30, 3.0) == 0.0
    assert np.isnan(f(-2.0, 2.5)) and np.isnan(f(float("nan"), 3.0))
    assert f(float("inf"), -2.0) == 0.0 and f(0.0, -1.0) == float("inf")
    # correctly rounded cubes of float-exact arguments, to within one unit in the last place
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(20000) * 10).astype(np.float32)
    got = np.array([f(float(v), 3.0) for v in x], dtype=np.float32)
    want = (x.astype(np.float64) ** 3).astype(np.float32)
    ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
    assert ulp.max() <= 1


def test_tanhf_matches_libm():
    """Every 521st float pattern (8.2 million arguments): the restated tanhf gives libm's bits (so does the full sweep
    of all 2^32 arguments, run once, for tanhf and for the expm1f it is built on)."""
    bad = C.c_uint32(0)
    n_bad = O.lib().orc_tanhf_count_mismatch(0, 0xFFFFFFFF, 521, C.byref(bad))
    assert n_bad == 0, (n_bad, hex(bad.value))


def test_tanhf_special_values():
    f = O.lib().orc_tanhf_det
    assert f(0.0) == 0.0 and math.copysign(1.0, f(-0.0)) == -1.0
    assert f(30.0) == 1.0 and f(-30.0) == -1.0 and f(float("inf")) == 1.0 and f(float("-inf")) == -1.0
    assert np.isnan(f(float("nan")))
    assert f(1e-20) == np.float32(1e-20)
    x = np.linspace(-12, 12, 4001).astype(np.float32)
    got = np.array([f(float(v)) for v in x], dtype=np.float32)
    want = np.tanh(x.astype(np.float64)).astype(np.float32)
    ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
    assert ulp.max() <= 2      # the float routine is accurate to about one unit in the last place, not correctly rounded
