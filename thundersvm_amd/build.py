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


def build_kernels(extra=(), only=None):
    """One object per source file, compiled side by side, then one link.  `only`: recompile just these sources and
    reuse the other objects of an earlier call (development)."""
    import concurrent.futures
    srcs = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    objdir = os.environ.get("TSVM_OBJ_DIR") or os.path.join(HERE, "build", "obj")   # (kept: `only` reuses the other objects)
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, f[:-4] + ".o") for f in srcs]
    todo = [(f, o) for f, o in zip(srcs, objs) if only is None or f in only or not os.path.exists(o)]
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(6, max(1, len(todo)))) as pool:
        list(pool.map(lambda fo: _run(["hipcc", *HIP_FLAGS, *extra, "-c", "-o", fo[1], os.path.join(CSRC, fo[0])]), todo))
    _run(["hipcc", *HIP_FLAGS, *extra, "-shared", "-o", KERNEL_LIB, *objs])
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


def build_selftests():
    """The test-only library (tests/native): self-tests of host-layer pieces, linked against the host library."""
    src = os.path.join(os.path.dirname(HERE), "tests", "native", "selftest.cpp")
    if not os.path.exists(src):
        return None
    out = os.path.join(os.path.dirname(src), "libtsvm_selftest.so")
    _run(["g++", "-O2", "-fPIC", "-std=c++17", "-fopenmp", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", src, "-shared", "-o", out,
          "-L", HERE, "-lthundersvm", "-ltsvm_hip", "-Wl,-rpath,$ORIGIN/../../thundersvm_amd", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"])
    return out


def build_all():
    build_kernels()
    build_host()
    build_selftests()


if __name__ == "__main__":
    build_all()
