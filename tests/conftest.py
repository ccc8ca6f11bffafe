import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

# The test session takes less than half of the device's memory for kernel rows: the driver clears what a process gives
# back before it hands it out again, and whoever asks for more than the untouched rest right afterwards waits for that
# (several seconds after a large arena).  With both halves below one half, the process that follows the tests does not.
os.environ.setdefault("TSVM_ARENA_PERCENT", "45")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
