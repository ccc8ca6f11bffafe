"""Reading and writing the LibSVM-compatible model text on the host (SvmModel::load_from_string / save_to_string,
src/thundersvm/model/svmmodel.cpp:193-383): the support-vector section is cut into runs of lines that several threads
read and write; the result is what one reader walking the lines in order gives.  Host only (no device call)."""
import numpy as np
import pytest

from thundersvm_amd.model import Model


def _model_text(n, k, rng, crlf=False):
    coef = rng.standard_normal((k - 1, n)) * 10.0 ** rng.integers(-6, 3, (k - 1, n))
    lines, cols, vals, ptr = [], [], [], [0]
    for i in range(n):
        nf = int(rng.integers(0, 9))
        c = np.sort(rng.choice(np.arange(1, 40), nf, replace=False))
        v = (rng.standard_normal(nf) * 10.0 ** rng.integers(-5, 4, nf)).astype(np.float32)
        v[rng.random(nf) < 0.3] = 1.0
        lines.append("".join("%.16g " % coef[j, i] for j in range(k - 1)) + "".join("%d:%.8g " % (a, b) for a, b in zip(c, v)))
        cols += list(c)
        vals += [float("%.8g" % b) for b in v]
        ptr.append(len(cols))
    per = [n // k + (1 if c < n % k else 0) for c in range(k)]
    head = ["svm_type c_svc", "kernel_type rbf", "gamma 0.25", "nr_class %d" % k, "total_sv %d" % n,
            "rho " + "".join("%.6g " % r for r in np.linspace(-1, 1, k * (k - 1) // 2)),
            "label " + "".join("%d " % (c + 1) for c in range(k)), "nr_sv " + "".join("%d " % p for p in per), "SV "]
    eol = "\r\n" if crlf else "\n"
    text = eol.join(head + lines) + eol
    want_coef = np.array([[float("%.16g" % coef[j, i]) for i in range(n)] for j in range(k - 1)])
    return text, want_coef, np.array(ptr), np.array(cols), np.array(vals)


@pytest.mark.parametrize("n,k", [(1, 2), (300, 2), (20000, 4)])
def test_load_then_save_gives_the_text_back(n, k, tmp_path):
    text, coef, ptr, cols, vals = _model_text(n, k, np.random.default_rng(n + k))
    path = str(tmp_path / "in.model")
    open(path, "w").write(text)
    m = Model(0)
    m.load(path)
    assert m.total_sv == n and m.n_classes == k
    assert np.array_equal(m.coef.reshape(k - 1, n), coef)
    assert np.array_equal(m.sv_ptr, ptr) and np.array_equal(m.sv_col, cols) and np.array_equal(m.sv_val, vals)
    out = str(tmp_path / "out.model")
    m.save(out)
    assert open(out).read() == text


def test_windows_line_ends_and_missing_lines(tmp_path):
    text, coef, ptr, cols, vals = _model_text(5000, 3, np.random.default_rng(5), crlf=True)
    path = str(tmp_path / "crlf.model")
    open(path, "w", newline="").write(text)
    m = Model(0)
    m.load(path)
    assert np.array_equal(m.coef.reshape(2, 5000), coef) and np.array_equal(m.sv_val, vals)
    # fewer lines than total_sv says: the missing support vectors are empty and their coefficients zero
    lines = text.replace("\r\n", "\n").split("\n")
    short = "\n".join(lines[:-101]) + "\n"          # the last 100 support-vector lines (and the final empty piece) are gone
    open(path, "w").write(short)
    m.load(path)
    assert m.total_sv == 5000 and np.array_equal(m.sv_ptr[-101:], np.full(101, ptr[-101]))
    assert np.array_equal(m.coef.reshape(2, 5000)[:, -100:], np.zeros((2, 100)))
    assert np.array_equal(m.coef.reshape(2, 5000)[:, :-100], coef[:, :-100])


def test_malformed_support_vector_line(tmp_path):
    from thundersvm_amd import capi
    text, *_ = _model_text(50, 2, np.random.default_rng(9))
    for bad in ("0.5 3;1 ", "0.5 3: ", "0.5 x:1 "):
        lines = text.split("\n")
        lines[-3] = bad
        path = str(tmp_path / "bad.model")
        open(path, "w").write("\n".join(lines))
        with pytest.raises(capi.TsvmError):
            Model(0).load(path)
