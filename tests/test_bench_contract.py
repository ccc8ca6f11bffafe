"""bench.py's command-line contract, as far as it can be checked without a device: more than one GPU is refused with a
message, and the loader-only mode (no device call) prints one JSON object with the text loader's figures."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused():
    r = _run("--gpus", "2")
    assert r.returncode == 2 and "exactly one GPU" in r.stderr and r.stdout == ""


def test_loader_only_prints_one_json_object():
    r = _run("--loader-only", "--workload", "c1")
    assert r.returncode == 0, r.stderr
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    assert out["file"]["rows"] == 3200 and out["file"]["bytes"] > 0
    for key in ("threads_1", "threads_all"):
        assert out["loader"][key]["seconds"] > 0 and out["loader"][key]["mb_per_s"] > 0
    assert out["loader"]["cores"] >= 1 and out["loader"]["speedup"] > 0
