"""Compiles libslowrun_ce.so (gfx950) in-tree with hipcc.

``python -m slowrun_amd.build`` or ``build_library()``.  The library is loaded by
``slowrun_amd._lib``; nothing is compiled at import time.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libslowrun_ce.so")
SOURCES = ["sce_kernels.hip", "sce_sort.hip"]
# packed fp32 math is kept off for every device function in this library
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]


def build_library(verbose=True, jobs=2):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    objs, procs = [], []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
        if len(procs) >= jobs:
            _wait(procs, verbose)
    _wait(procs, verbose)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


def build_abi_example(verbose=True):
    """tests/abi_example.c -> tests/bin/abi_example: a plain C caller of the library (gcc, no hipcc), linked against
    libslowrun_ce.so and the HIP runtime.  Run by tests/test_c_abi.py on a GPU."""
    root = os.path.dirname(HERE)
    out_dir = os.path.join(root, "tests", "bin")
    os.makedirs(out_dir, exist_ok=True)
    exe = os.path.join(out_dir, "abi_example")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-std=c11", "-O2", "-Wall", "-D__HIP_PLATFORM_AMD__", f"-I{rocm}/include", f"-I{os.path.join(root, 'include')}",
           os.path.join(root, "tests", "abi_example.c"), "-o", exe, f"-L{rocm}/lib", "-lamdhip64", f"-L{HERE}", "-lslowrun_ce", "-lm",
           "-Wl,-rpath,$ORIGIN/../../slowrun_amd", f"-Wl,-rpath,{rocm}/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return exe


def _wait(procs, verbose):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out, flush=True)


if __name__ == "__main__":
    print(build_library())
    print(build_abi_example())
    sys.exit(0)
