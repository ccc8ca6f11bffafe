"""The LibSVM-compatible model text, byte for byte (SvmModel::save_to_string, src/thundersvm/model/svmmodel.cpp:193-264).

The expected files under tests/golden/ were written by hand from the reference's writer and the closed form of each
two-point problem, not by running this library:

* field order: svm_type, kernel_type, [degree], [gamma], [coef0], nr_class, total_sv, rho, [label, nr_sv], [probA, probB],
  [coef + the linear coefficients], SV and one line per support vector;
* every list element is followed by one blank, also the last one of a line ("rho -0 ", "SV ", "coef ");
* numbers go through an ostream in its default floating-point format: 6 significant digits for gamma, coef0, rho, probA /
  probB; setprecision(16) for coefficients and linear coefficients; setprecision(8) for support-vector values.

The problems (every step below is exact in binary floating point unless it says otherwise):

model_csvc_rbf_two_points.txt -- rows  3 1:0.123456789 3:-2.5  and  -7 1:-1 2:1e-05, RBF gamma = 0.123456789, C = 0.25.
  The first local step moves both alphas by min(C, C, 2 / (2 - 2 K12)) = 0.25 (K12 < 1), after which neither is free.
  Coefficients are alpha * y = 0.25 and -0.25.  f1 = -0.75 - 0.25 K12 and f2 = 0.75 + 0.25 K12, so
  rho = -(f2 + f1) / 2 = -(+0) / 2 = -0.  gamma prints with 6 digits (0.123457); the values are the floats the loader made
  of the text, printed with 8 digits: 0.123456789 -> 0.12345679, 1e-05 -> 9.9999997e-06.
model_svr_rbf_two_points.txt -- rows  2.125 1:1  and  -1 1:-1, epsilon-SVR with p = 0.5, C = 0.25, gamma = 0.5.
  The doubled problem starts from f = (p - y1, p - y2, -p - y1, -p - y2) = (-1.625, 1.5, -2.625, 0.5); the only step
  pairs variable 0 with variable 3 and moves both to C.  Coefficients alpha_i - alpha_{i+n} = 0.25 and -0.25;
  rho = -((0.25 + 0.25 K12) + (-1.375 - 0.25 K12)) / 2 = 0.5625.  No label / nr_sv lines for a regression model.
model_csvc_linear_two_points.txt -- rows  1 1:1 2:0.5  and  -1 1:-1 2:0.25, linear kernel, C = 1/3.
  K11 = 1.25, K22 = 1.0625, K12 = -0.875; the step is min(C, C, 2 / 4.0625) = C.  Coefficients +-0.3333333333333333
  (16 digits); linear coefficients C*1 + C*1 = 0.6666666666666666 and C*0.5 - C*0.25 = C/4 = 0.08333333333333333;
  rho = -((1 - 1.9375 C) + (-1 + 2.125 C)) / 2 = -0.03125 up to a rounding error far below the 6 printed digits.
"""
import os

import numpy as np
import pytest

from thundersvm_amd import data as D
from thundersvm_amd.model import Model, make_param

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _rows(text, tmp_path):
    path = str(tmp_path / "train.txt")
    open(path, "w").write(text)
    return D.load_libsvm(path)


CASES = {
    "model_csvc_rbf_two_points.txt": ("3 1:0.123456789 3:-2.5\n-7 1:-1 2:1e-05\n",
                                      dict(svm_type=0, kernel_type=2, gamma=0.123456789, C=0.25)),
    "model_svr_rbf_two_points.txt": ("2.125 1:1\n-1 1:-1\n", dict(svm_type=3, kernel_type=2, gamma=0.5, C=0.25, p=0.5)),
    "model_csvc_linear_two_points.txt": ("1 1:1 2:0.5\n-1 1:-1 2:0.25\n", dict(svm_type=0, kernel_type=0, C=1.0 / 3.0)),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_saved_model_text_byte_for_byte(name, tmp_path):
    text, prm = CASES[name]
    tr = _rows(text, tmp_path)
    m = Model(prm["svm_type"]).train(tr, make_param(**prm))
    out = str(tmp_path / "out.model")
    m.save(out)
    got = open(out, "rb").read()
    want = open(os.path.join(GOLDEN, name), "rb").read()
    assert got == want, "\n--- got ---\n%s--- want ---\n%s" % (got.decode(), want.decode())
    # the text loads back into a model that writes the same text and predicts the same values
    again = Model(prm["svm_type"]).load(out)
    out2 = str(tmp_path / "out2.model")
    again.save(out2)
    assert open(out2, "rb").read() == want
    _, dec = m.predict(tr)
    _, dec2 = again.predict(tr)
    assert np.abs(dec - dec2).max() < 1e-6       # (values went through 8 digits, rho through 6)


def test_libsvm_style_model_with_double_values(tmp_path):
    """A model as LibSVM itself would write it: no blank at the end of a line, rho with 17 digits, support-vector values
    that are not floats.  The reference reads them with "%d:%lf" in a double build (svmmodel.cpp:362-366): every digit
    arrives, and prediction uses them."""
    path = os.path.join(GOLDEN, "model_libsvm_style_double_values.txt")
    m = Model(0).load(path)
    assert m.total_sv == 3 and m.n_sv.tolist() == [2, 1] and m.label.tolist() == [1, -1]
    assert m.rho[0] == 0.12345678901234567
    assert m.coef.tolist() == [0.75, 0.25, -1.0]
    assert m.sv_ptr.tolist() == [0, 2, 3, 5] and m.sv_col.tolist() == [1, 2, 2, 1, 3]
    assert m.sv_val.tolist() == [0.1234567890123456, 1.0, -0.30000000000000004, 1.0, 2.0000000000000004]
    # decision values from the closed form: sum coef * expf(-gamma |x - sv|^2) - rho, the kernel value a float
    x = np.array([[0.5, -0.25, 1.0], [0.0, 0.0, 0.0], [1.0, 0.0, 2.0]])
    sv = np.array([[0.1234567890123456, 1.0, 0.0], [0.0, -0.30000000000000004, 0.0], [1.0, 0.0, 2.0000000000000004]])
    want = []
    for r in x:
        k = [float(np.exp(np.float32(-0.5 * ((r - s) ** 2).sum())).astype(np.float32)) for s in sv]
        want.append(0.75 * k[0] + 0.25 * k[1] - 1.0 * k[2] - 0.12345678901234567)
    lab, dec = m.predict(D.from_dense(x, np.zeros(3), keep_zeros=False))
    assert np.abs(dec[:, 0] - np.array(want)).max() < 1e-6
    assert lab.tolist() == [1.0 if v > 0 else -1.0 for v in want]


def test_support_vector_lines_of_a_large_model(tmp_path):
    """The support-vector lines are written by several threads, runs of lines each; joined they are the lines a single
    writer makes: every coefficient with 16 significant digits, every value with 8, in the model's own order."""
    rng = np.random.default_rng(12)
    k, per, d = 4, 900, 6
    centres = rng.standard_normal((k, d))
    cls = rng.permutation(np.repeat(np.arange(k), per))
    x = (centres[cls] + 1.2 * rng.standard_normal((k * per, d))).astype(np.float32)
    x[rng.random(x.shape) < 0.3] = 0.0                      # rows of different lengths
    tr = D.from_dense(x, (cls + 1).astype(np.float64))
    m = Model(0).train(tr, make_param(svm_type=0, kernel_type=2, gamma=0.4, C=2.0))
    assert m.total_sv > 2000                                # many runs of 256 lines and more
    out = str(tmp_path / "big.model")
    m.save(out)
    lines = open(out).read().split("\n")
    start = lines.index("SV ") + 1
    body = lines[start:]
    assert body[-1] == "" and len(body) == m.total_sv + 1
    coef = m.coef.reshape(k - 1, m.total_sv)
    for i in range(m.total_sv):
        lo, hi = m.sv_ptr[i], m.sv_ptr[i + 1]
        want = "".join("%.16g " % coef[j, i] for j in range(k - 1))
        want += "".join("%d:%.8g " % (c, v) for c, v in zip(m.sv_col[lo:hi], m.sv_val[lo:hi]))
        assert body[i] == want, i
    # and the text loads back to the same model text
    m2 = Model(0)
    m2.load(out)
    out2 = str(tmp_path / "big2.model")
    m2.save(out2)
    assert open(out2).read() == open(out).read()
