"""Pins oracle/eager.py and oracle/closed_form.py against one another and
against what the mathematics fixes.  The reference has no tests or golden
vectors for this path, so these are the anchors:

* closed_form (explicit formulas, numpy float64)  vs  eager (torch autograd)
* closed_form.backward  vs  central finite differences of closed_form.forward
* cap -> infinity  ==  F.cross_entropy on the raw logits (library routine)
* W = 0  =>  loss == ln V exactly, dX == 0
* sum_v dz_iv == 0 on valid rows; ignored rows give a zero dX row and do not
  count in the mean; all rows ignored => NaN mean (F.cross_entropy's 0/0)
* row permutation permutes losses / dX and leaves dW unchanged
* scaling X and x_s by 2 leaves the fp8 bytes unchanged (and doubles the logits)
* chunked evaluation == unchunked
* MTP: n_predict = 1 equals the plain path bit for bit; weights [1,0,0] == [1]
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import closed_form, eager


def _tiny(seed=0, N=12, d=16, V=40, ignore=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, d, generator=g, dtype=torch.float64)
    w = torch.randn(d, V, generator=g, dtype=torch.float64) * 0.7
    y = torch.randint(0, V, (N,), generator=g)
    if ignore:
        y[1] = -1
        y[N - 2] = -1
    return x, w, y


def test_closed_form_vs_eager_autograd_fp64_mean():
    x, w, y = _tiny()
    cap = 3.0
    o = eager.softcapped_ce(x, w, y, cap=cap, reduction="mean", dtype=torch.float64, row_chunk=5)
    loss, b = closed_form.mean_loss_and_grads(x.numpy(), w.numpy(), y.numpy(), cap)
    assert abs(float(o["loss"]) - loss) < 1e-12
    np.testing.assert_allclose(o["dx"].numpy(), b["dx"], rtol=0, atol=1e-13)
    np.testing.assert_allclose(o["dw"].numpy(), b["dw"], rtol=0, atol=1e-13)
    np.testing.assert_allclose(o["lse"].numpy(), b["lse"], rtol=0, atol=1e-12)
    assert np.array_equal(o["argmax"].numpy(), b["argmax"])


def test_closed_form_vs_eager_none_with_upstream():
    x, w, y = _tiny(seed=1)
    cap = 2.0
    g = torch.rand(x.shape[0], dtype=torch.float64, generator=torch.Generator().manual_seed(5))
    o = eager.softcapped_ce(x, w, y, cap=cap, reduction="none", grad_output=g, dtype=torch.float64)
    b = closed_form.backward(x.numpy(), w.numpy(), y.numpy(), cap, g.numpy())
    np.testing.assert_allclose(o["loss"].numpy(), b["losses"], atol=1e-12)
    assert o["loss"][1] == 0 and o["loss"][-2] == 0          # ignored rows report 0
    np.testing.assert_allclose(o["dx"].numpy(), b["dx"], atol=1e-13)
    np.testing.assert_allclose(o["dw"].numpy(), b["dw"], atol=1e-13)


def test_closed_form_backward_vs_finite_differences():
    x, w, y = _tiny(seed=2, N=6, d=5, V=9)
    x, w, y = x.numpy(), w.numpy(), y.numpy()
    cap = 1.7
    rng = np.random.default_rng(0)
    g = rng.random(x.shape[0])
    b = closed_form.backward(x, w, y, cap, g)

    def total(xx, ww):
        return float((closed_form.forward(xx, ww, y, cap)["losses"] * g).sum())

    eps = 1e-6
    for arr, grad, which in ((x, b["dx"], 0), (w, b["dw"], 1)):
        num = np.zeros_like(arr)
        for idx in np.ndindex(arr.shape):
            hi = arr.copy(); hi[idx] += eps
            lo = arr.copy(); lo[idx] -= eps
            num[idx] = (total(hi, w) - total(lo, w)) / (2 * eps) if which == 0 else \
                (total(x, hi) - total(x, lo)) / (2 * eps)
        np.testing.assert_allclose(grad, num, rtol=1e-6, atol=1e-8)


def test_mtp_closed_form_vs_finite_differences_and_eager():
    x, w, y = _tiny(seed=3, N=7, d=4, V=8)
    cap = 2.5
    wts = (1.0, 0.5, 0.25)
    rng = np.random.default_rng(1)
    g = rng.random(x.shape[0])
    b = closed_form.backward(x.numpy(), w.numpy(), y.numpy(), cap, g, wts)
    o = eager.softcapped_ce_mtp(x, w, y, wts, cap=cap, grad_output=torch.from_numpy(g), dtype=torch.float64)
    np.testing.assert_allclose(o["loss"].numpy(), b["losses"], atol=1e-12)
    np.testing.assert_allclose(o["dx"].numpy(), b["dx"], atol=1e-13)
    np.testing.assert_allclose(o["dw"].numpy(), b["dw"], atol=1e-13)
    eps = 1e-6
    xn = x.numpy()
    num = np.zeros_like(xn)
    for idx in np.ndindex(xn.shape):
        hi = xn.copy(); hi[idx] += eps
        lo = xn.copy(); lo[idx] -= eps
        num[idx] = ((closed_form.forward(hi, w.numpy(), y.numpy(), cap, wts)["losses"] * g).sum()
                    - (closed_form.forward(lo, w.numpy(), y.numpy(), cap, wts)["losses"] * g).sum()) / (2 * eps)
    np.testing.assert_allclose(b["dx"], num, rtol=1e-6, atol=1e-8)


def test_cap_to_infinity_is_plain_cross_entropy():
    x, w, y = _tiny(seed=4)
    o = eager.softcapped_ce(x, w, y, cap=1e9, reduction="mean", dtype=torch.float64)
    xl = x.clone().requires_grad_(True)
    wl = w.clone().requires_grad_(True)
    ref = F.cross_entropy(xl @ wl, y, ignore_index=-1)
    ref.backward()
    assert abs(float(o["loss"]) - float(ref.detach())) < 1e-9
    np.testing.assert_allclose(o["dx"].numpy(), xl.grad.numpy(), atol=1e-9)
    np.testing.assert_allclose(o["dw"].numpy(), wl.grad.numpy(), atol=1e-9)
    loss, b = closed_form.mean_loss_and_grads(x.numpy(), w.numpy(), y.numpy(), 1e9)
    assert abs(loss - float(ref.detach())) < 1e-9


def test_saturated_rows_have_vanishing_gradient():
    # |u| >> cap: z -> +-cap and 1 - tanh^2 -> 0
    x, w, y = _tiny(seed=5, ignore=False)
    b = closed_form.backward((x * 500).numpy(), w.numpy(), y.numpy(), 1.0, np.ones(x.shape[0]))
    assert np.abs(b["z"]).max() <= 1.0 and np.median(np.abs(b["z"])) > 0.999999
    sat = np.abs(b["u"]) > 20.0
    assert sat.mean() > 0.9 and np.abs(b["du"][sat]).max() < 1e-15


def test_zero_weight_gives_ln_v():
    x, w, y = _tiny(seed=6, ignore=False)
    V = w.shape[1]
    o = eager.softcapped_ce(x, torch.zeros_like(w), y, cap=15.0, reduction="mean", dtype=torch.float64)
    assert abs(float(o["loss"]) - math.log(V)) < 1e-12
    assert float(o["dx"].abs().max()) == 0.0
    b = closed_form.forward(x.numpy(), np.zeros_like(w.numpy()), y.numpy(), 15.0)
    np.testing.assert_allclose(b["losses"], math.log(V), atol=1e-12)


def test_dz_rows_sum_to_zero_and_ignored_rows():
    x, w, y = _tiny(seed=7)
    loss, b = closed_form.mean_loss_and_grads(x.numpy(), w.numpy(), y.numpy(), 4.0)
    np.testing.assert_allclose(b["dz"].sum(axis=1), 0, atol=1e-15)
    assert np.all(b["dx"][1] == 0) and np.all(b["dx"][-2] == 0)
    # the mean is over valid rows only
    valid = y.numpy() != -1
    assert abs(loss - b["losses"][valid].mean()) < 1e-14
    # dropping the ignored rows changes nothing
    loss2, b2 = closed_form.mean_loss_and_grads(x.numpy()[valid], w.numpy(), y.numpy()[valid], 4.0)
    assert abs(loss - loss2) < 1e-14
    np.testing.assert_allclose(b["dw"], b2["dw"], atol=1e-15)


def test_all_ignored_mean_is_nan_like_torch():
    x, w, y = _tiny(seed=8)
    y[:] = -1
    ref = F.cross_entropy(x @ w, y, ignore_index=-1)
    assert math.isnan(float(ref))
    o = eager.softcapped_ce(x, w, y, cap=15.0, reduction="mean", dtype=torch.float64)
    assert math.isnan(float(o["loss"]))
    assert float(o["dx"].abs().max()) == 0 and float(o["dw"].abs().max()) == 0
    o2 = eager.softcapped_ce(x, w, y, cap=15.0, reduction="none", dtype=torch.float64)
    assert float(o2["loss"].abs().max()) == 0


def test_row_permutation_equivariance():
    x, w, y = _tiny(seed=9)
    perm = torch.randperm(x.shape[0], generator=torch.Generator().manual_seed(1))
    a = eager.softcapped_ce(x, w, y, cap=5.0, reduction="none", dtype=torch.float64)
    b = eager.softcapped_ce(x[perm], w, y[perm], cap=5.0, reduction="none", dtype=torch.float64)
    np.testing.assert_allclose(a["loss"][perm].numpy(), b["loss"].numpy(), atol=1e-13)
    np.testing.assert_allclose(a["dx"][perm].numpy(), b["dx"].numpy(), atol=1e-14)
    np.testing.assert_allclose(a["dw"].numpy(), b["dw"].numpy(), atol=1e-14)


def test_quantised_scale_invariance_and_chunking():
    g = torch.Generator().manual_seed(10)
    x = torch.randn(64, 32, generator=g)
    w = torch.randn(32, 96, generator=g) * 0.2
    y = torch.randint(0, 96, (64,), generator=g)
    x_s = float(x.abs().max()) / 448
    w_s = float(w.abs().max()) / 448
    a = eager.softcapped_ce(x, w, y, x_s, w_s, cap=15.0, row_chunk=64)
    # scaling X and x_s by the same power of two leaves the fp8 bytes unchanged, so the
    # quantised path on (2X, 2x_s) is the unquantised path on twice the dequantised X
    assert torch.equal(eager.quantize_e4m3(x, x_s).view(torch.uint8), eager.quantize_e4m3(2 * x, 2 * x_s).view(torch.uint8))
    b = eager.softcapped_ce(2 * x, w, y, 2 * x_s, w_s, cap=15.0, row_chunk=64)
    xq = eager.dequantize(eager.quantize_e4m3(x, x_s), x_s)
    wq = eager.dequantize(eager.quantize_e4m3(w, w_s), w_s)
    b2 = eager.softcapped_ce(2 * xq, wq, y, None, None, cap=15.0, row_chunk=64)
    assert float(b["loss"]) == float(b2["loss"])
    assert torch.equal(b["dx"], b2["dx"]) and torch.equal(b["dw"], b2["dw"])
    c = eager.softcapped_ce(x, w, y, x_s, w_s, cap=15.0, row_chunk=7)
    assert abs(float(a["loss"]) - float(c["loss"])) < 1e-6
    # a row's logits do not depend on which chunk it sits in, but the fp32 matmul
    # may block differently: allow rounding-level differences only
    np.testing.assert_allclose(a["dx"].numpy(), c["dx"].numpy(), atol=1e-7)
    np.testing.assert_allclose(a["dw"].numpy(), c["dw"].numpy(), atol=1e-6)


def test_quantised_eager_uses_dequantised_fp8_values():
    # The matmul must see deq(fp8(x / s)) * s, not x: compare with closed_form on those values
    from oracle import fp8
    g = torch.Generator().manual_seed(11)
    x = torch.randn(10, 16, generator=g)
    w = torch.randn(16, 24, generator=g) * 0.3
    y = torch.randint(0, 24, (10,), generator=g)
    x_s, w_s = 100 / 448, 1.6 / 448                      # the reference's fixed scales (tiny/train.py:188-189)
    xq = fp8.decode_e4m3(fp8.encode_e4m3((x / torch.tensor(x_s)).numpy())) * np.float32(x_s)
    wq = fp8.decode_e4m3(fp8.encode_e4m3((w / torch.tensor(w_s)).numpy())) * np.float32(w_s)
    loss, b = closed_form.mean_loss_and_grads(xq, wq, y.numpy(), 15.0)
    o = eager.softcapped_ce(x, w, y, x_s, w_s, cap=15.0)
    assert abs(float(o["loss"]) - loss) < 1e-5
    np.testing.assert_allclose(o["dx"].numpy(), b["dx"], atol=1e-6)
    np.testing.assert_allclose(o["dw"].numpy(), b["dw"], atol=1e-6)


def test_mtp_single_offset_is_plain_path():
    x, w, y = _tiny(seed=12)
    x, w = x.float(), w.float()
    a = eager.softcapped_ce(x, w, y, cap=15.0, reduction="none")
    b = eager.softcapped_ce_mtp(x, w, y, [1.0], cap=15.0)
    c = eager.softcapped_ce_mtp(x, w, y, [1.0, 0.0, 0.0], cap=15.0)
    assert torch.equal(a["loss"], b["loss"]) and torch.equal(a["dx"], b["dx"]) and torch.equal(a["dw"], b["dw"])
    assert torch.equal(a["loss"], c["loss"]) and torch.equal(a["dx"], c["dx"]) and torch.equal(a["dw"], c["dw"])


def test_mtp_with_fewer_rows_than_offsets():
    """One or two rows and four offsets: the offsets beyond the last row take no part, so the result is that of the
    offsets that have a row."""
    x, w, y = _tiny(seed=13)
    x, w = x.float(), w.float()
    for n in (1, 2):
        a = eager.softcapped_ce_mtp(x[:n], w, y[:n], [1.0, 0.5, 0.25, 0.125], cap=15.0)
        b = eager.softcapped_ce_mtp(x[:n], w, y[:n], [1.0, 0.5][:n], cap=15.0)
        assert torch.equal(a["loss"], b["loss"]) and torch.equal(a["dx"], b["dx"]) and torch.equal(a["dw"], b["dw"])


def test_mtp_reference_kernel_formula_on_valid_targets():
    # tiny/cuda_kernels.py:226-240: loss_i = sum_k w_k (lse_i - z[i, y_{i+k}]) for i + k < N
    x, w, y = _tiny(seed=13, ignore=False)
    cap = 15.0
    wts = [1.0, 0.5, 0.25]
    f = closed_form.forward(x.numpy(), w.numpy(), y.numpy(), cap)
    N = x.shape[0]
    want = np.zeros(N)
    for i in range(N):
        for k, wk in enumerate(wts):
            if i + k < N:
                want[i] += wk * (f["lse"][i] - f["z"][i, y[i + k]])
    o = eager.softcapped_ce_mtp(x, w, y, wts, cap=cap, dtype=torch.float64)
    np.testing.assert_allclose(o["loss"].numpy(), want, atol=1e-12)


def test_rms_norm_restatement_vs_library_and_autograd():
    """oracle.eager.rms_norm / rms_norm_backward against F.rms_norm and its autograd gradient (fp32 and fp64)."""
    g = torch.Generator().manual_seed(5)
    h = torch.randn(37, 48, generator=g) * 2.5
    x, rstd = eager.rms_norm(h)
    assert torch.equal(x, F.rms_norm(h, (48,)))
    x2, _ = eager.rms_norm(h, eps=1e-3)
    assert torch.equal(x2, F.rms_norm(h, (48,), eps=1e-3))
    hd = h.double().requires_grad_(True)
    up = torch.randn(37, 48, generator=g, dtype=torch.float64)
    F.rms_norm(hd, (48,), eps=1e-3).backward(up)
    _, rstd64 = eager.rms_norm(h.double(), eps=1e-3)
    ours = eager.rms_norm_backward(h.double(), rstd64.double(), up)
    # float() inside the restatement limits this to fp32 accuracy
    assert (ours.double() - hd.grad).abs().max() < 1e-5 * hd.grad.abs().max()
    # bf16 input: fp32 arithmetic, float32's epsilon by default, a single rounding: bit-identical to the library
    hb = (torch.randn(300, 2560, generator=g) * 3).bfloat16()
    assert torch.equal(eager.rms_norm(hb)[0], F.rms_norm(hb, (2560,)))
    assert torch.equal(eager.rms_norm(hb, eps=1e-6)[0], F.rms_norm(hb, (2560,), eps=1e-6))
