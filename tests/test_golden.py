"""Committed golden vectors (tests/golden/ce_small.npz, written by
tests/golden/make_fixtures.py from the float64 closed form on table-quantised
fp8 values).  CPU: the torch oracle must reproduce them, which ties
oracle/eager.py (library cast, matmul, autograd) to oracle/closed_form.py +
oracle/fp8.py on stored data.  GPU: the HIP path must reproduce them."""
import os

import numpy as np
import pytest
import torch

from oracle import eager

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ce_small.npz"))
CASES = sorted({k.split("/")[0] for k in FIX.files})


def _case(name):
    return {k.split("/")[1]: FIX[k] for k in FIX.files if k.startswith(name + "/")}


@pytest.mark.parametrize("name", CASES)
def test_oracle_reproduces_golden(name):
    c = _case(name)
    x = torch.from_numpy(c["x"]).bfloat16()
    w = torch.from_numpy(c["w"]).bfloat16()
    y = torch.from_numpy(c["y"])
    x_s, w_s, cap = float(c["x_s"]), float(c["w_s"]), float(c["cap"])
    assert np.array_equal(eager.quantize_e4m3(x, x_s).view(torch.uint8).numpy(), c["xq_codes"])
    assert np.array_equal(eager.quantize_e4m3(w, w_s).view(torch.uint8).numpy(), c["wq_codes"])
    o = eager.softcapped_ce(x, w, y, x_s, w_s, cap=cap, reduction="mean", dtype=torch.float64)
    # the oracle dequantises in float32 (code * scale rounded once), the fixture in float64
    assert abs(float(o["loss"]) - float(c["loss"])) < 1e-6
    np.testing.assert_allclose(o["lse"].numpy(), c["lse"], atol=1e-6)
    np.testing.assert_allclose(o["dx"].numpy(), c["dx"], atol=1e-6 * np.abs(c["dx"]).max())
    np.testing.assert_allclose(o["dw"].numpy(), c["dw"], atol=1e-6 * np.abs(c["dw"]).max())
    assert np.array_equal(o["argmax"].numpy(), c["argmax"])


@pytest.mark.gpu
@pytest.mark.parametrize("keep", [False, True])
@pytest.mark.parametrize("name", CASES)
def test_hip_path_reproduces_golden(name, keep):
    """keep: the forward pass emits the dlogits (the default of the autograd Function) / backward computes them again."""
    from slowrun_amd import cuda_kernels as ck
    from tests import parity_util as pu
    c = _case(name)
    x = torch.from_numpy(c["x"]).cuda().bfloat16()
    w = torch.from_numpy(c["w"]).cuda().bfloat16()
    y = torch.from_numpy(c["y"]).cuda()
    N, d = x.shape
    V = w.shape[1]
    x_s, w_s, cap = float(c["x_s"]), float(c["w_s"]), float(c["cap"])
    assert np.array_equal(ck.quantize_e4m3(x, x_s).view(torch.uint8).cpu().numpy(), c["xq_codes"])
    assert np.array_equal(ck.quantize_e4m3(w, w_s).view(torch.uint8).cpu().numpy(), c["wq_codes"])
    loss, saved, lse, argmax, n_valid = ck.ce_forward(x, w, y, x_s, w_s, cap, "mean", want_argmax=True, keep_dlogits=keep)
    dx, dw = ck.ce_backward(saved, y, torch.ones((), device="cuda"), N, d, V, x_s, w_s, cap, 1.0, "mean",
                            torch.float32, torch.float32, keep_dlogits=keep)
    assert abs(float(loss) - float(c["loss"])) / abs(float(c["loss"])) < pu.LOSS_RTOL
    np.testing.assert_allclose(lse.cpu().numpy(), c["lse"], rtol=1e-5, atol=1e-5)
    assert np.array_equal(argmax.cpu().numpy().astype(np.int64), c["argmax"])
    assert int(n_valid[0]) == int((c["y"] != -1).sum())
    for got, ref in ((dx, c["dx"]), (dw, c["dw"])):
        ref = torch.from_numpy(ref)
        assert pu.maxrel(got.cpu(), ref) <= pu.GRAD_MAXREL and pu.cosine(got.cpu(), ref) > pu.GRAD_COS
    ign = torch.from_numpy(c["y"] == -1)
    if ign.any():
        assert float(dx.cpu()[ign].abs().max()) == 0.0
