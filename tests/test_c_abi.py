"""The C ABI without Python in between: tests/abi_example.c, a plain C program that includes only
include/slowrun_ce.h and the HIP runtime, is built ahead of time by slowrun_amd/build.py and run here."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "bin", "abi_example")


@pytest.fixture(scope="module")
def exe():
    """The prebuilt program; built here only when nothing is there (hipcc and gcc work without a GPU)."""
    from slowrun_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build_library(verbose=False)
    if not os.path.exists(EXE):
        build.build_abi_example(verbose=False)
    return EXE


def test_example_is_built_and_linked_against_the_library(exe):
    out = subprocess.run(["ldd", exe], capture_output=True, text=True, check=True).stdout
    line = [l for l in out.splitlines() if "libslowrun_ce.so" in l]
    assert line and "not found" not in line[0], out
    assert os.path.realpath(line[0].split("=>")[1].split("(")[0].strip()) == os.path.realpath(
        os.path.join(ROOT, "slowrun_amd", "libslowrun_ce.so"))


@pytest.mark.gpu
def test_c_caller_matches_double_precision_formulas(exe):
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "abi_example: ok" in r.stdout
