"""ctypes binding of libslowrun_ce.so (C ABI in include/slowrun_ce.h).

The library is the only compute path: if it is missing or cannot be loaded the
import of this module's ``lib()`` raises, there is no fallback.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libslowrun_ce.so")

SCE_F32, SCE_BF16 = 0, 1
SCE_REDUCE_NONE, SCE_REDUCE_MEAN = 0, 1
SCE_VERSION = 4

EXPORTS = ("sce_version", "sce_last_error", "sce_sizes_for", "sce_quantize_e4m3", "sce_quantize_e4m3_dev", "sce_amax_scale",
           "sce_transpose_bytes",
           "sce_forward", "sce_forward_noalloc", "sce_backward", "sce_timing_enable", "sce_timing_read", "sce_bench_mfma", "sce_bench_gemm", "sce_bench_floor",
           "sce_test_set_gather_limit")

KERNEL_KINDS = ("quantize", "fwd", "fwd_reduce", "bwd_prep", "recompute", "dx", "dw", "dw_final")


class SceShape(C.Structure):
    _fields_ = [("N", C.c_int64), ("d", C.c_int64), ("V", C.c_int64), ("n_predict", C.c_int32), ("reserved", C.c_int32)]


class SceSizes(C.Structure):
    _fields_ = [("saved_bytes", C.c_size_t), ("saved_x_bytes", C.c_size_t), ("wcache_bytes", C.c_size_t),
                ("fwd_workspace_bytes", C.c_size_t),
                ("bwd_workspace_min_bytes", C.c_size_t), ("bwd_workspace_bytes", C.c_size_t),
                ("bwd_panel_rows", C.c_int64), ("dlogits_bytes", C.c_size_t), ("bwd_workspace_kept_bytes", C.c_size_t), ("saved_bf16_bytes", C.c_size_t)]


class SceArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("device", C.c_int32), ("stream", C.c_void_p), ("shape", SceShape),
        ("x", C.c_void_p), ("x_dtype", C.c_int32), ("pad0", C.c_int32), ("x_ld", C.c_int64),
        ("w", C.c_void_p), ("w_dtype", C.c_int32), ("pad1", C.c_int32), ("w_ld", C.c_int64),
        ("targets", C.c_void_p), ("mtp_weights", C.c_void_p),
        ("x_s", C.c_double), ("w_s", C.c_double), ("cap", C.c_float), ("grad_scale", C.c_float),
        ("ignore_index", C.c_int64), ("reduction", C.c_int32), ("pad2", C.c_int32),
        ("loss", C.c_void_p), ("losses", C.c_void_p), ("lse", C.c_void_p), ("argmax", C.c_void_p), ("n_valid", C.c_void_p),
        ("saved", C.c_void_p), ("saved_bytes", C.c_size_t), ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("grad_output", C.c_void_p),
        ("dx", C.c_void_p), ("dx_dtype", C.c_int32), ("pad3", C.c_int32), ("dx_ld", C.c_int64),
        ("dw", C.c_void_p), ("dw_dtype", C.c_int32), ("pad4", C.c_int32), ("dw_ld", C.c_int64),
        ("panel_rows", C.c_int64),
        ("vocab_limit", C.c_int64), ("wcache", C.c_void_p), ("wcache_bytes", C.c_size_t),
        ("wcache_valid", C.c_int32), ("norm", C.c_int32), ("norm_eps", C.c_float), ("dlogits_from_forward", C.c_int32),
        ("x_s_dev", C.c_void_p), ("w_s_dev", C.c_void_p), ("operand_dtype", C.c_int32), ("pad6", C.c_int32),
    ]


class SceTiming(C.Structure):
    _fields_ = [("ms", C.c_double * 8), ("launches", C.c_int64 * 8)]


_LIB = None


def lib():
    """Load the shared library once; raise if it is not there."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m slowrun_amd.build` (needs hipcc); "
                "there is no fallback path")
        L = C.CDLL(LIB_PATH)
        L.sce_version.restype = C.c_int
        L.sce_last_error.restype = C.c_char_p
        L.sce_sizes_for.argtypes = [C.POINTER(SceShape), C.POINTER(SceSizes)]
        L.sce_quantize_e4m3.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_double, C.c_size_t, C.c_int32, C.c_void_p]
        L.sce_quantize_e4m3_dev.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int32, C.c_void_p]
        L.sce_amax_scale.argtypes = [C.c_void_p, C.c_int32, C.c_size_t, C.c_void_p, C.c_int32, C.c_void_p]
        L.sce_transpose_bytes.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.c_void_p]
        L.sce_forward.argtypes = [C.POINTER(SceArgs)]
        L.sce_forward_noalloc.argtypes = [C.POINTER(SceArgs)]
        L.sce_backward.argtypes = [C.POINTER(SceArgs)]
        L.sce_bench_mfma.argtypes = [C.c_void_p, C.c_size_t, C.c_int32, C.c_int32, C.c_void_p, C.c_size_t, C.c_int32, C.c_void_p,
                                     C.POINTER(C.c_double), C.POINTER(C.c_double)]
        L.sce_bench_gemm.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_size_t,
                                     C.c_int32, C.c_void_p, C.POINTER(C.c_double), C.POINTER(C.c_double)]
        L.sce_bench_floor.argtypes = [C.POINTER(SceArgs), C.c_int32, C.c_int32, C.c_void_p, C.c_size_t, C.POINTER(C.c_double), C.POINTER(C.c_double)]
        L.sce_test_set_gather_limit.restype = C.c_int64
        L.sce_test_set_gather_limit.argtypes = [C.c_int64]
        L.sce_timing_enable.argtypes = [C.c_int]
        L.sce_timing_read.argtypes = [C.POINTER(SceTiming)]
        if L.sce_version() != SCE_VERSION:
            raise RuntimeError(f"libslowrun_ce.so has ABI version {L.sce_version()}, expected {SCE_VERSION}")
        _LIB = L
    return _LIB


def check(rc, what):
    if rc != 0:
        msg = lib().sce_last_error().decode()
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")


def sizes_for(N, d, V, n_predict=1):
    shape = SceShape(N, d, V, n_predict, 0)
    out = SceSizes()
    check(lib().sce_sizes_for(C.byref(shape), C.byref(out)), "sce_sizes_for")
    return out


def timing_enable(on):
    check(lib().sce_timing_enable(1 if on else 0), "sce_timing_enable")


def timing_read():
    """{kind: (total_ms, launches)} accumulated since timing_enable(True)."""
    t = SceTiming()
    check(lib().sce_timing_read(C.byref(t)), "sce_timing_read")
    return {k: (t.ms[i], t.launches[i]) for i, k in enumerate(KERNEL_KINDS)}
