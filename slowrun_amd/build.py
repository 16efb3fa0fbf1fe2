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
    warn_if_other_toolchain()
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


# The toolchain the hand-scheduled parts of the kernels were written and measured against: the main loop's direct-to-LDS
# loads write M0 inside inline asm (the compiler refuses the register as a clobber) and count their own s_waitcnt vmcnt,
# and the register allocation of the 256-accumulator kernels decides whether anything is spilled around the main loop.
# Another compiler may well be fine; kernel_resources() and the GPU tests are what tells.
TESTED_HIPCC = "7.2.26015"


def hipcc_version():
    """The 'HIP version' line of `hipcc --version` ('' if it cannot be run)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    try:
        out = subprocess.run([hipcc, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True).stdout
    except OSError:
        return ""
    for ln in out.splitlines():
        if ln.startswith("HIP version:"):
            return ln.split(":", 1)[1].strip()
    return ""


def warn_if_other_toolchain():
    v = hipcc_version()
    if v and not v.startswith(TESTED_HIPCC):
        print(f"slowrun_amd.build: warning: hipcc reports HIP version {v}; the kernels' hand-placed waits and register budgets were "
              f"checked with {TESTED_HIPCC}.  Run `python -m slowrun_amd.build --resources` and the GPU tests before trusting results.",
              file=sys.stderr, flush=True)
    return v


_RES_KEYS = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch", "Occupancy [waves/SIMD]": "occupancy",
             "SGPRs Spill": "sgpr_spill", "VGPRs Spill": "vgpr_spill", "LDS Size [bytes/block]": "lds"}


def kernel_resources(verbose=False):
    """{demangled kernel name: {sgprs, vgprs, agprs, scratch, occupancy, sgpr_spill, vgpr_spill, lds}} of every kernel in
    sce_kernels.hip, from the compiler's own remarks (-Rpass-analysis=kernel-resource-usage; device code only, nothing is
    linked or written)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, *HIP_FLAGS, "--cuda-device-only", "-c", os.path.join(CSRC, "sce_kernels.hip"), "-o", os.devnull,
           "-Rpass-analysis=kernel-resource-usage"]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out.stdout)
    res, cur = {}, None
    for ln in out.stdout.splitlines():
        if "remark:" not in ln:
            continue
        body = ln.split("remark:", 1)[1].replace("[-Rpass-analysis=kernel-resource-usage]", "").strip()
        key, _, val = body.partition(":")
        key, val = key.strip(), val.strip()
        if key == "Function Name":
            cur = res.setdefault(val, {})
        elif cur is not None and key in _RES_KEYS:
            cur[_RES_KEYS[key]] = int(val)
    names = list(res)
    filt = shutil.which("c++filt") or shutil.which("llvm-cxxfilt") or "c++filt"
    try:
        dem = subprocess.run([filt], input="\n".join(names), stdout=subprocess.PIPE, text=True, check=True).stdout.splitlines()
    except (OSError, subprocess.CalledProcessError):
        dem = names
    table = {}
    for m, dname in zip(names, dem):
        short = dname.split("(")[0].replace("sce::", "").replace("void ", "").strip()
        table[short] = res[m]
    return table


def format_resources(table):
    rows = [f"{'kernel':48s} {'VGPR':>5s} {'AGPR':>5s} {'SGPR':>5s} {'SGPR spill':>10s} {'VGPR spill':>10s} {'scratch B/lane':>14s} {'waves/SIMD':>10s} {'LDS B':>7s}"]
    for k in sorted(table):
        r = table[k]
        rows.append(f"{k:48s} {r['vgprs']:5d} {r['agprs']:5d} {r['sgprs']:5d} {r['sgpr_spill']:10d} {r['vgpr_spill']:10d} {r['scratch']:14d} {r['occupancy']:10d} {r['lds']:7d}")
    return "\n".join(rows)


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
    if "--resources" in sys.argv[1:]:
        print(f"hipcc HIP version {hipcc_version()}")
        print(format_resources(kernel_resources(verbose=True)))
        sys.exit(0)
    print(build_library())
    print(build_abi_example())
    sys.exit(0)
