"""The reference trainer's call of the loss head as one unit, at its real size: tiny/train.py:682-696 flattens a device
batch of 32 x 2048 tokens at d = 1024 and calls FusedSoftcappedCrossEntropy.apply(x, targets, mtp_weights, W, 100/448,
1.6/448, 0.75/448, 1.0) with three prediction offsets (tiny/train.py:125,186-193); the result is reduced with .mean()
and differentiated (tiny/train.py:1417-1419).  Checked against the eager restatement evaluated row-chunked with stock
torch on the same device and the same bf16 inputs, in both backward modes."""
import pytest
import torch

from slowrun_amd import configs
from tests import parity_util as pu

pytestmark = pytest.mark.gpu

MTP_X_S, MTP_W_S, MTP_GRAD_S = 100 / 448, 1.6 / 448, 0.75 / 448       # tiny/train.py:188-190


@pytest.mark.parametrize("keep", [True, False])
def test_trainer_call_at_full_size(keep):
    from oracle import eager
    from slowrun_amd.cuda_kernels import CE_KERNEL_VOCAB_SIZE, FusedSoftcappedCrossEntropy
    N, d, V = 65536, 1024, CE_KERNEL_VOCAB_SIZE
    weights = [1.0, 0.5, 0.25]
    inp = configs.make_inputs("tiny_track", N=N)
    assert inp.shape == (N, d, V)
    x = inp.x.cuda().bfloat16().requires_grad_(True)
    w = inp.w.cuda().bfloat16().requires_grad_(True)
    y = inp.targets.cuda()
    mw = torch.tensor(weights, device="cuda")
    losses = FusedSoftcappedCrossEntropy.apply(x, y, mw, w, MTP_X_S, MTP_W_S, MTP_GRAD_S, 1.0, 15.0, "none", keep)
    assert losses.shape == (N,) and losses.dtype == torch.float32
    losses.mean().backward()
    torch.cuda.synchronize()
    assert x.grad.dtype == torch.bfloat16 and w.grad.dtype == torch.bfloat16
    ref = eager.softcapped_ce_mtp(x.detach(), w.detach(), y, weights, MTP_X_S, MTP_W_S, cap=15.0, row_chunk=2048)   # grad_output = 1 / N
    rel = float((losses.detach() - ref["loss"]).abs().max() / ref["loss"].abs().max())
    rel_mean = abs(float(losses.detach().double().mean()) - float(ref["loss"].double().mean())) / float(ref["loss"].double().mean())
    rep = {"loss_rel_max": rel, "mean_loss_rel": rel_mean}
    for name, got, want in (("dx", x.grad, ref["dx"]), ("dw", w.grad, ref["dw"])):
        rep[name + "_maxrel"], rep[name + "_cos"] = pu.maxrel(got.float(), want), pu.cosine(got.float(), want)
    print("trainer call", "keep" if keep else "recompute", rep)
    assert rel <= pu.LOSS_RTOL and rel_mean <= pu.LOSS_RTOL
    for name in ("dx", "dw"):
        assert rep[name + "_maxrel"] <= pu.GRAD_MAXREL and rep[name + "_cos"] > pu.GRAD_COS
    # the last rows have fewer offsets (they would run past the end of the flattened targets): still finite, still positive
    assert bool(torch.isfinite(losses).all()) and float(losses[-1]) > 0


def test_backward_with_flags_that_differ_from_forward_gives_nan_not_wrong_numbers():
    """sce_backward reads the state sce_forward left.  Asked for something else than the forward call was (dlogits kept or not,
    another vocabulary limit), that state does not fit: every gradient comes out NaN instead of silently wrong."""
    from slowrun_amd import cuda_kernels as ck
    inp = configs.make_inputs("tiny_track", N=512, d=128, V=1024)
    x, w, y = inp.x.cuda().bfloat16(), inp.w.cuda().bfloat16(), inp.targets.cuda()
    N, d, V = inp.shape
    go = torch.ones((), device="cuda")
    _loss, saved, _lse, _am, _nv = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "mean", keep_dlogits=False)
    args = (saved, y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.float32, torch.float32)
    dx, dw = ck.ce_backward(*args, keep_dlogits=False)
    assert bool(torch.isfinite(dx).all()) and bool(torch.isfinite(dw).all())
    dx, dw = ck.ce_backward(*args, keep_dlogits=False, vocab_size=1000)               # forward used all 1024 columns
    assert bool(torch.isnan(dx).all()) and bool(torch.isnan(dw).all())
    big = torch.zeros(saved.numel() + ck._lib.sizes_for(N, d, V).dlogits_bytes, dtype=torch.uint8, device="cuda")
    big[: saved.numel()] = saved
    dx, dw = ck.ce_backward(big, *args[1:], keep_dlogits=True)                        # forward emitted no dlogits
    assert bool(torch.isnan(dx).all()) and bool(torch.isnan(dw).all())
