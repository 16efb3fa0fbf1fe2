"""The C ABI without a GPU: the library loads, exports every function the header
declares, the ctypes mirror of the structs matches the C layout, and argument
validation fails with the documented codes and messages (no kernel is launched)."""
import ctypes as C
import os
import re
import subprocess

import pytest

from slowrun_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "slowrun_ce.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from slowrun_amd import build
        build.build_library(verbose=False)
    return _lib.lib()


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sce_[a-z0-9_]+)\s*\(", text)))


def test_header_functions_are_exported(lib):
    names = _declared_functions()
    assert set(names) == set(_lib.EXPORTS), (names, _lib.EXPORTS)
    for n in names:
        assert getattr(lib, n) is not None          # raises AttributeError if the symbol is missing


def test_version(lib):
    assert lib.sce_version() == _lib.SCE_VERSION == 4


def test_struct_layout_matches_c(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "%s"\n'
                   'int main(void){ printf("%%zu %%zu %%zu %%zu %%zu %%zu %%zu %%zu\\n", sizeof(sce_args), offsetof(sce_args, shape),'
                   ' offsetof(sce_args, targets), offsetof(sce_args, saved), offsetof(sce_args, grad_output),'
                   ' offsetof(sce_args, panel_rows), sizeof(sce_sizes), sizeof(sce_timing)); return 0; }\n' % HEADER)
    exe = tmp_path / "layout"
    subprocess.run(["gcc", str(src), "-o", str(exe)], check=True)
    got = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    A = _lib.SceArgs
    want = [C.sizeof(A), A.shape.offset, A.targets.offset, A.saved.offset, A.grad_output.offset, A.panel_rows.offset,
            C.sizeof(_lib.SceSizes), C.sizeof(_lib.SceTiming)]
    assert got == want


def test_sizes_for_and_shape_errors(lib):
    s = _lib.sizes_for(65536, 2560, 50304)
    # X_q + W_q^T + W_q in e4m3 (rows padded by 128 bytes) plus four per-row statistics: nothing N x V sized is kept for backward
    assert s.saved_bytes < (65536 + 50432) * (2560 + 128) + 2560 * (50432 + 128) + 5 * 65536 * 4
    assert s.bwd_workspace_min_bytes <= s.bwd_workspace_bytes
    assert s.bwd_panel_rows % 256 == 0 and s.bwd_panel_rows * 10 <= 256 * 256
    for bad in [(0, 128, 100), (10, 100, 100), (10, 128, 0), (1 << 25, 128, 100)]:
        with pytest.raises(RuntimeError):
            _lib.sizes_for(*bad)
    # the largest vocabulary: the block exponents of one dX tile's K loop (V / 128 blocks) wait in LDS behind the K slots
    assert _lib.sizes_for(256, 64, 524288).dlogits_bytes == 524288 * 256 + 4096 * 2 * 4
    with pytest.raises(RuntimeError, match="at most 524288"):
        _lib.sizes_for(256, 64, 524288 + 64)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        _lib.sizes_for(256, 72, 1000)
    with pytest.raises(RuntimeError, match="below 2\\^24"):
        _lib.sizes_for((1 << 24) - 100, 64, 1000)
    shape = _lib.SceShape(10, 128, 100, 5, 0)          # at most 4 multi-token-prediction offsets
    out = _lib.SceSizes()
    assert lib.sce_sizes_for(C.byref(shape), C.byref(out)) == 1
    assert b"n_predict" in lib.sce_last_error()
    assert lib.sce_sizes_for(None, C.byref(out)) == 1


def test_argument_validation_without_gpu(lib):
    a = _lib.SceArgs()
    assert lib.sce_forward(None) == 1 and b"NULL" in lib.sce_last_error()
    a.struct_size = 12
    assert lib.sce_forward(C.byref(a)) == 1 and b"struct_size" in lib.sce_last_error()
    a.struct_size = C.sizeof(_lib.SceArgs)
    a.shape = _lib.SceShape(256, 128, 512, 1, 0)
    assert lib.sce_forward(C.byref(a)) == 1 and b"targets" in lib.sce_last_error()
    a.targets = 256
    a.cap, a.x_s, a.w_s = 100.0, 1.0, 1.0
    assert lib.sce_backward(C.byref(a)) == 1 and b"cap" in lib.sce_last_error()
    a.cap, a.x_s = 15.0, 0.0
    assert lib.sce_forward(C.byref(a)) == 1 and b"x_s" in lib.sce_last_error()
    assert lib.sce_quantize_e4m3(None, 0, None, 1.0, 16, 0, None) == 1
    assert lib.sce_transpose_bytes(None, None, 4, 4, 0, None) == 1
    t = _lib.SceTiming()
    assert lib.sce_timing_enable(0) == 0 and lib.sce_timing_read(C.byref(t)) == 0 and sum(t.launches) == 0


def test_python_wrapper_refuses_cpu_tensors():
    import torch
    from slowrun_amd.cuda_kernels import FusedSoftcappedCrossEntropy
    x = torch.randn(8, 16)
    w = torch.randn(16, 32)
    y = torch.randint(0, 32, (8,))
    with pytest.raises(RuntimeError, match="GPU"):
        FusedSoftcappedCrossEntropy.apply(x, y, None, w, 1.0, 1.0, 1.0, 1.0)


def test_custom_ops_have_fake_implementations():
    """torch.compile traces the loss head through slowrun_amd::ce_forward / ce_backward; their fake
    implementations must give the shapes and dtypes of the real ones (checked here on meta tensors)."""
    import torch
    from slowrun_amd import cuda_kernels as ck
    x = torch.empty(512, 128, dtype=torch.bfloat16, device="meta")
    w = torch.empty(128, 1024, dtype=torch.bfloat16, device="meta")
    y = torch.empty(512, dtype=torch.int64, device="meta")
    mw = torch.empty(3, dtype=torch.float32, device="meta")
    out, saved = ck.ce_forward_op(x, w, y, mw, 0.1, 0.1, 15.0, False, False)
    assert out.shape == (512,) and out.dtype == torch.float32
    sz3 = _lib.sizes_for(512, 128, 1024, 3)
    assert saved.dtype == torch.uint8 and saved.numel() == sz3.saved_bytes
    out2, saved2 = ck.ce_forward_op(x, w, y, mw, 0.1, 0.1, 15.0, True, True)         # the dlogits travel in `saved`
    assert out2.shape == () and saved2.numel() == sz3.saved_bytes + sz3.dlogits_bytes and sz3.dlogits_bytes >= 512 * 1024
    dx, dw = ck.ce_backward_op(saved, y, out, mw, 512, 128, 1024, 0.1, 0.1, 15.0, 1.0, False, True, False, False)
    assert dx.shape == (512, 128) and dx.dtype == torch.bfloat16 and dw.shape == (128, 1024) and dw.dtype == torch.float32
    out3, saved3 = ck.norm_ce_forward_op(x, w, y, None, 0.1, 0.1, 15.0, True, 1e-6, False)
    assert out3.shape == () and saved3.numel() == _lib.sizes_for(512, 128, 1024, 1).saved_bytes
    dh, dw2 = ck.norm_ce_backward_op(saved3, x, y, out3, None, 1024, 0.1, 0.1, 15.0, 1.0, True, True, 1e-6, False)
    assert dh.shape == (512, 128) and dh.dtype == torch.bfloat16 and dw2.shape == (128, 1024) and dw2.dtype == torch.bfloat16


def test_error_messages_are_per_thread(lib):
    """sce_last_error is thread-local: concurrent callers that fail in different ways each read their own message."""
    import threading
    results = {}

    def worker(tag, shape_args, needle):
        ok = True
        for _ in range(200):
            shape = _lib.SceShape(*shape_args)
            out = _lib.SceSizes()
            rc = lib.sce_sizes_for(C.byref(shape), C.byref(out))
            ok = ok and rc == 1 and needle in lib.sce_last_error()
        results[tag] = ok

    threads = [threading.Thread(target=worker, args=("d", (10, 100, 100, 1, 0), b"multiple of 16")),
               threading.Thread(target=worker, args=("k", (10, 128, 100, 7, 0), b"n_predict")),
               threading.Thread(target=worker, args=("n", (0, 128, 100, 1, 0), b"positive"))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert results == {"d": True, "k": True, "n": True}
