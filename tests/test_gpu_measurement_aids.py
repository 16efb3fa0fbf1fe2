"""The measurement aids of the C ABI (sce_bench_mfma, sce_bench_gemm; slowrun_amd.ceiling builds its
report from them): they run at small sizes, return figures that make sense for this part, and refuse shapes their
kernels do not take."""
import ctypes as C

import pytest
import torch

from slowrun_amd import _lib, ceiling

pytestmark = pytest.mark.gpu


def _scratch():
    return torch.empty(64 << 20, dtype=torch.uint8, device="cuda")


def test_matrix_instruction_alone():
    scratch = _scratch()
    tf_const, mhz_const = ceiling._mfma(False, scratch, iters=2000, reps=2)
    tf_rand, mhz_rand = ceiling._mfma(True, scratch, iters=2000, reps=2)
    # constant operands reach the published rate at the full clock; random operands are slower, never faster
    assert 0.5 * ceiling.PEAK_FP8_TFLOPS < tf_const < 1.05 * ceiling.PEAK_FP8_TFLOPS
    assert 1000 < mhz_rand <= mhz_const * 1.02 < 2600
    assert 0.3 * ceiling.PEAK_FP8_TFLOPS < tf_rand < tf_const * 1.02


def test_main_loop_alone():
    scratch = _scratch()
    tf, mhz = ceiling._gemm(4096, 4096, 2048, "random", scratch, reps=3)
    assert 500 < tf < ceiling.PEAK_FP8_TFLOPS and 1000 < mhz < 2600


def test_shapes_the_kernels_do_not_take_are_refused():
    scratch = _scratch()
    lib = _lib.lib()
    a = ceiling._operand(4096, 1024, "zero", scratch.device)
    tf, mhz = C.c_double(), C.c_double()
    args = (scratch.data_ptr(), scratch.numel(), scratch.device.index, None)
    assert lib.sce_bench_gemm(a.data_ptr(), a.data_ptr(), 4096, 4000, 1024, 1, *args, C.byref(tf), C.byref(mhz)) == 1
    assert b"multiples of 256" in lib.sce_last_error()
    assert lib.sce_bench_gemm(None, a.data_ptr(), 4096, 4096, 1024, 1, *args, C.byref(tf), C.byref(mhz)) == 1
    assert lib.sce_bench_mfma(None, 0, 0, 1, *args, C.byref(tf), C.byref(mhz)) == 1
    assert lib.sce_bench_mfma(a.data_ptr(), 4096, 10, 1, *args, C.byref(tf), C.byref(mhz)) == 1      # operand bytes too few
    assert b"random_bytes" in lib.sce_last_error()
    assert lib.sce_bench_gemm(a.data_ptr(), a.data_ptr(), 4096, 4096, 1024, 1, scratch.data_ptr(), 16, scratch.device.index, None,
                              C.byref(tf), C.byref(mhz)) == 1                                                       # scratch too small
