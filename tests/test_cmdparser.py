"""Command-line parsing of thundersvm-train, after src/test/test_cmd.cpp:36-189: every flag, the
defaults of SvmParam, the default model-file name and rejection of invalid values."""
import ctypes as C
import os
import subprocess

import pytest

from thundersvm_amd import model
from thundersvm_amd.model import TsvmParam

BIN = os.path.join(os.path.dirname(model.__file__), "bin")


def parse(*args):
    argv = ["thundersvm-train"] + list(args)
    arr = (C.c_char_p * len(argv))(*[a.encode() for a in argv])
    prm = TsvmParam()
    gs, cv, nf = C.c_int(), C.c_int(), C.c_int()
    inp, mod = C.create_string_buffer(256), C.create_string_buffer(256)
    L = model.host_lib()
    L.tsvm_cmdparser_train.argtypes = [C.c_int, C.POINTER(C.c_char_p), C.POINTER(TsvmParam), C.POINTER(C.c_int),
                                       C.POINTER(C.c_int), C.POINTER(C.c_int), C.c_char_p, C.c_char_p, C.c_int]
    rc = L.tsvm_cmdparser_train(len(argv), arr, C.byref(prm), C.byref(gs), C.byref(cv), C.byref(nf), inp, mod, 256)
    return rc, prm, gs.value, cv.value, nf.value, inp.value.decode(), mod.value.decode()


def test_defaults():
    rc, p, gs, cv, nf, inp, mod = parse("dataset/test_dataset.txt")
    assert rc == 0
    assert (p.svm_type, p.kernel_type, p.degree) == (0, 2, 3)
    assert p.C == 1 and p.gamma == 0 and p.coef0 == 0 and p.nu == 0.5
    assert abs(p.p - 0.1) < 1e-7 and abs(p.epsilon - 0.001) < 1e-9
    assert p.max_mem_size == 8192 << 20
    assert not gs and not cv
    assert inp == "dataset/test_dataset.txt" and mod == "test_dataset.txt.model"


def test_all_flags():
    rc, p, gs, cv, nf, inp, mod = parse("-s", "3", "-t", "1", "-d", "5", "-g", "1/8", "-r", "0.25", "-c", "10", "-n", "0.3",
                                        "-p", "0.2", "-m", "1024", "-e", "0.01", "-w1", "2.5", "-w-1", "0.5", "-v", "5", "-q",
                                        "train.txt", "out.model")
    assert rc == 0
    assert (p.svm_type, p.kernel_type, p.degree) == (3, 1, 5)
    assert p.gamma == 0.125 and p.coef0 == 0.25 and p.C == 10 and p.nu == 0.3 and p.p == 0.2 and p.epsilon == 0.01
    assert p.max_mem_size == 1024 << 20 and p.nr_weight == 2 and p.verbose == 0
    assert gs and cv and nf == 5 and inp == "train.txt" and mod == "out.model"


@pytest.mark.parametrize("args", [["-s", "7", "f"], ["-t", "9", "f"], ["-g", "-1", "f"], ["-e", "0", "f"], ["-c", "-2", "f"],
                                  ["-s", "1", "-n", "1.5", "f"], ["-v", "1", "f"], ["-z", "1", "f"], ["-c"], []])
def test_invalid(args):
    rc = parse(*args)[0]
    assert rc == -1
    assert model.host_lib().tsvm_model_last_error()


def test_executable_usage():
    exe = os.path.join(BIN, "thundersvm-train")
    if not os.path.exists(exe):
        pytest.skip("CLI not built")
    r = subprocess.run([exe, "-s", "9", "x"], capture_output=True, text=True)
    assert r.returncode == 1 and "Usage: thundersvm-train" in r.stderr


@pytest.mark.gpu
def test_train_predict_cli(tmp_path):
    fixture = os.path.join(os.path.dirname(__file__), "golden", "test_dataset.txt")
    mfile, out = str(tmp_path / "m.model"), str(tmp_path / "pred.txt")
    r = subprocess.run([os.path.join(BIN, "thundersvm-train"), "-c", "100", "-g", "0.5", fixture, mfile], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert "all training time" in r.stderr
    text = open(mfile).read()
    assert text.startswith("svm_type c_svc\nkernel_type rbf\ngamma 0.5\nnr_class 3\ntotal_sv ")
    assert "label 0 2 3 \n" in text
    r = subprocess.run([os.path.join(BIN, "thundersvm-predict"), fixture, mfile, out], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert "Accuracy = 0.98" in r.stderr                       # README.md:95-98 of the reference
    labels = [float(v) for v in open(out).read().split()]
    assert len(labels) == 150
