"""The LibSVM text loader of the host layer (DataSet::load_from_file, the reference's src/thundersvm/dataset.cpp:20-100):
parsing on many threads gives what one thread gives -- values, row order, labels, the zero-based flag, the feature
count -- and both give what a straightforward Python parse with numpy's float32 rounding gives.  Host only."""
import os

import numpy as np
import pytest

from thundersvm_amd import data as D
from thundersvm_amd.model import Dataset

FIXTURE = os.path.join(os.path.dirname(__file__), "golden", "test_dataset.txt")


def _same(a, b):
    (ca, nfa, za), (cb, nfb, zb) = a, b
    assert nfa == nfb and za == zb
    assert np.array_equal(ca.ptr, cb.ptr) and np.array_equal(ca.col, cb.col)
    assert np.array_equal(ca.val.view(np.int64), cb.val.view(np.int64))      # bit for bit
    assert np.array_equal(ca.y, cb.y)


def _against_python(path, loaded):
    csr, nf, zb = loaded
    ref = D.load_libsvm(path)
    assert np.array_equal(csr.ptr, ref.ptr) and np.array_equal(csr.col, ref.col)
    assert np.array_equal(csr.val, ref.val) and np.array_equal(csr.y, ref.y)
    assert nf == (int(ref.col.max()) if len(ref.col) else 0) and zb == bool((ref.col == 0).any())


def test_reference_fixture():
    one = Dataset(path=FIXTURE, threads=1).csr()
    _against_python(FIXTURE, one)
    assert one[0].n == 150 and one[1] == 4
    for t in (2, 3, 8, 16, 0):
        _same(one, Dataset(path=FIXTURE, threads=t).csr())


def test_seven_class_workload_text(tmp_path):
    """The multi-class benchmark's text at a reduced row count: 10 continuous features written with nine digits and two
    one-hot blocks."""
    tr = D.workload_c4(scale=0.02)["train"]
    path = str(tmp_path / "c4.txt")
    D.save_libsvm(path, tr)
    one = Dataset(path=path, threads=1).csr()
    assert np.array_equal(one[0].ptr, tr.ptr) and np.array_equal(one[0].col, tr.col)
    assert np.array_equal(one[0].val, tr.val) and np.array_equal(one[0].y, tr.y)
    for t in (2, 5, 16):
        _same(one, Dataset(path=path, threads=t).csr())
    # without the last newline the last row is still there
    text = open(path).read()
    assert text.endswith("\n")
    open(path, "w").write(text[:-1])
    for t in (1, 7):
        _same(one, Dataset(path=path, threads=t).csr())


def test_number_forms_and_layout(tmp_path):
    """Every way a LibSVM file writes a number goes through float exactly once (sscanf %f in the reference): long
    decimal tails, exponents, values that a detour through double would round the other way, denormal floats, huge and
    tiny exponents, signs, a zero-based index, Windows line ends, blank lines, leading blanks, tabs."""
    rng = np.random.default_rng(3)
    tokens = ["0.1", "-0.1", "+2.5", "1e-3", "1E+5", "3.4028235e38", "1e-45", "1.17549435e-38", "7e-46", "123456789012345678901234",
              "0.000000000000000000000000000001", "1.00000005960464477539062500001", "1.000000059604644775390625",
              "16777217", "16777219.0000000001", "0", "-0", "00012.5000", ".5", "5.", "1e0", "9007199254740993", "4.35e-5",
              "8.589973e9", "0.30000001192092896", "1.4e-45", "3e38"]
    tokens += ["%.17g" % v for v in rng.standard_normal(200) * 10.0 ** rng.integers(-8, 8, 200)]
    tokens += ["%.9g" % v for v in rng.standard_normal(200).astype(np.float32)]
    # midpoints between neighbouring floats, written exactly and a hair to either side
    for f in rng.standard_normal(40).astype(np.float32):
        up = np.nextafter(f, np.float32(np.inf))
        mid = (float(f) + float(up)) / 2
        tokens += ["%.30g" % mid, "%.25g" % (mid * (1 + 1e-15)), "%.25g" % (mid * (1 - 1e-15))]
    lines, k = [], 0
    while k < len(tokens):
        take = int(rng.integers(1, 9))
        feats = " ".join("%d:%s" % (j + (0 if k == 0 else 1), t) for j, t in enumerate(tokens[k:k + take]))
        lines.append("%s %s" % (["1", "-1", "2.5", "1e1", "+3"][len(lines) % 5], feats))
        k += take
    lines[3] = "  \t" + lines[3].replace(" ", "\t", 1) + "  "
    text = "\r\n".join(lines[:10]) + "\r\n\n\n" + "\n".join(lines[10:]) + "\n"
    path = str(tmp_path / "numbers.txt")
    open(path, "w").write(text)
    one = Dataset(path=path, threads=1).csr()
    assert one[0].n == len(lines) and one[2] is True
    # expected values: the decimal text rounded once to float (numpy parses the text to double exactly-rounded, and
    # float(text) -> float32 can round twice, so the expectation is built from exact rational arithmetic)
    from fractions import Fraction
    def to_f32(tok):
        v = Fraction(tok) if "e" not in tok.lower() else Fraction(tok.lower().split("e")[0]) * Fraction(10) ** int(tok.lower().split("e")[1])
        if v == 0:
            return np.float32(-0.0 if tok.startswith("-") else 0.0)
        d = np.float32(float(v))                       # a candidate, within one float of the right answer
        if not np.isfinite(d):
            return d
        with np.errstate(over="ignore"):
            cands = [np.nextafter(d, np.float32(-np.inf)), d, np.nextafter(d, np.float32(np.inf))]
        cands = [c for c in cands if np.isfinite(c)]
        best = min(cands, key=lambda c: (abs(Fraction(float(c)) - v), int(np.float32(c).view(np.int32)) & 1))
        big = Fraction(float(np.finfo(np.float32).max)) + Fraction(2) ** 103      # beyond this a float rounds to infinity
        return np.float32(np.inf) * (1 if v > 0 else -1) if abs(v) >= big else best
    want = np.array([float(to_f32(t)) for t in tokens])
    assert np.array_equal(one[0].val.view(np.int64), want.view(np.int64))
    for t in (2, 4, 16):
        _same(one, Dataset(path=path, threads=t).csr())


def test_file_that_ends_on_a_page_boundary(tmp_path):
    """The file is parsed from a mapping of its pages: a file whose size is a whole number of pages has nothing behind
    its last byte, so a last line without a newline must not be handed to a library call that reads on (its last token
    here is one the short decimal parser leaves to strtof: 25 digits)."""
    page = os.sysconf("SC_PAGE_SIZE")
    last = "-1 1:0.5 3:1.000000059604644775390625"
    for final_newline in (False, True):
        body = "".join("1 1:%d.25 2:%d\n" % (i, i % 7) for i in range(3000))
        end = last + ("\n" if final_newline else "")
        pad = (-(len(body) + len(end))) % page
        assert pad == 0 or pad >= 8
        if pad:
            body += "2 5:" + "0" * (pad - 6) + "1\n"        # a line of exactly `pad` bytes
        text = body + end
        assert len(text) % page == 0
        path = str(tmp_path / ("page_%d.txt" % final_newline))
        open(path, "w").write(text)
        one = Dataset(path=path, threads=1).csr()
        _against_python(path, one)
        assert one[0].n == 3000 + (1 if pad else 0) + 1 and one[0].y[-1] == -1.0
        assert one[0].val[-1] == 1.0      # 1 + 2^-24, the midpoint between two floats, rounds to the even one
        for t in (3, 16):
            _same(one, Dataset(path=path, threads=t).csr())


def test_bad_input(tmp_path):
    from thundersvm_amd import capi
    path = str(tmp_path / "bad.txt")
    open(path, "w").write("1 1:0.5 2;0.25\n")
    with pytest.raises(capi.TsvmError):
        Dataset(path=path, threads=2)
    with pytest.raises(capi.TsvmError):
        Dataset(path=str(tmp_path / "missing.txt"))
    open(path, "w").write("")
    assert Dataset(path=path, threads=4).n == 0
