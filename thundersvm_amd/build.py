"""Builds the gfx950 kernel library (libtsvm_hip.so) and the host C++ library in-tree with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
KERNEL_LIB = os.path.join(HERE, "libtsvm_hip.so")
HOST_LIB = os.path.join(HERE, "libthundersvm.so")

HIP_FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-value",
             "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument"]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_kernels(extra=()):
    srcs = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))
    _run(["hipcc", *HIP_FLAGS, *extra, "-shared", "-o", KERNEL_LIB, *srcs])
    return KERNEL_LIB


def build_host(extra=()):
    if not os.path.isdir(HOST):
        return None
    srcs = sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cpp") and not f.startswith("main_"))
    if not srcs:
        return None
    _run(["g++", "-O2", "-fPIC", "-std=c++17", "-ffp-contract=off", "-fopenmp", "-D__HIP_PLATFORM_AMD__",
          "-I/opt/rocm/include", *extra, *srcs, "-shared", "-o", HOST_LIB,
          "-L", HERE, "-ltsvm_hip", "-Wl,-rpath,$ORIGIN", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"])
    for main in sorted(f for f in os.listdir(HOST) if f.startswith("main_") and f.endswith(".cpp")):
        exe = os.path.join(HERE, "bin", main[len("main_"):-len(".cpp")].replace("_", "-"))
        os.makedirs(os.path.dirname(exe), exist_ok=True)
        _run(["g++", "-O2", "-std=c++17", "-fopenmp", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
              os.path.join(HOST, main), "-o", exe, "-L", HERE, "-lthundersvm", "-ltsvm_hip",
              "-Wl,-rpath,$ORIGIN/..", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"])
    return HOST_LIB


def build_all():
    build_kernels()
    build_host()


if __name__ == "__main__":
    build_all()
