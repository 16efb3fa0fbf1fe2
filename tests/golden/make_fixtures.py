"""Writes tests/golden/ce_small.npz: seeded small inputs and float64 expected outputs.

The expected values come from oracle/closed_form.py (explicit formulas, numpy
float64) applied to the fp8 values produced by oracle/fp8.py (table-based e4m3
encode/decode), i.e. without torch's cast, matmul or autograd.  Nothing from the
reference is imported or run.  Regenerate with:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import closed_form, fp8  # noqa: E402


def bf16_round(a):
    """Round float32 to the nearest bfloat16 (ties to even), returned as float32."""
    u = np.asarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def main():
    rng = np.random.default_rng(20240607)
    cases = {}
    for name, (N, d, V, cap, n_ign, xmul) in {
        "plain": (96, 64, 320, 15.0, 0, 1.0),
        "ignored_and_saturated": (70, 48, 200, 4.0, 9, 6.0),
    }.items():
        x = rng.standard_normal((N, d)).astype(np.float32)
        x /= np.sqrt((x * x).mean(axis=1, keepdims=True))
        x = bf16_round(x * xmul)
        w = bf16_round((rng.standard_normal((d, V)) * d ** -0.5).astype(np.float32))
        y = rng.integers(0, V, N).astype(np.int64)
        if n_ign:
            y[rng.choice(N, n_ign, replace=False)] = -1
        x_s = np.float32(np.abs(x).max() / 448.0)
        w_s = np.float32(np.abs(w).max() / 448.0)
        # quantise as the reference does on bf16 tensors: fp32 quotient, rounded to bf16, cast to e4m3
        xq_codes = fp8.encode_e4m3(bf16_round(x / x_s))
        wq_codes = fp8.encode_e4m3(bf16_round(w / w_s))
        xq = fp8.decode_e4m3(xq_codes) * np.float64(x_s)
        wq = fp8.decode_e4m3(wq_codes) * np.float64(w_s)
        loss, b = closed_form.mean_loss_and_grads(xq, wq, y, cap)
        cases[name] = dict(x=x, w=w, y=y, x_s=x_s, w_s=w_s, cap=np.float64(cap), xq_codes=xq_codes, wq_codes=wq_codes,
                           loss=np.float64(loss), losses=b["losses"], lse=b["lse"], argmax=b["argmax"].astype(np.int64),
                           dx=b["dx"], dw=b["dw"])
    flat = {f"{c}/{k}": v for c, d_ in cases.items() for k, v in d_.items()}
    np.savez_compressed(os.path.join(HERE, "ce_small.npz"), **flat)
    print("wrote", os.path.join(HERE, "ce_small.npz"), {k: v.shape for k, v in flat.items() if hasattr(v, "shape")})


if __name__ == "__main__":
    main()
