"""GPU parity of the ping-pong forward kernel (fwd_pp_kernel, selected with SCE_FWD_KERNEL=pingpong): the same checks
against the oracle as the default kernel gets, and agreement with the default kernel on what the two must share."""
import pytest
import torch

from oracle import eager
from slowrun_amd import configs
from tests import parity_util as pu
from tests.test_gpu_parity_peaked import make_peaked, per_row_rel

pytestmark = pytest.mark.gpu


@pytest.fixture
def pingpong(monkeypatch):
    monkeypatch.setenv("SCE_FWD_KERNEL", "pingpong")


# one row tile and one column tile; both sides of the tile boundaries; a short K loop; more than one V split; the tiny-track width
SHAPES = [(256, 128, 256), (300, 128, 1000), (1000, 80, 777), (513, 272, 2049), (64, 16, 50304), (700, 1024, 9000)]


@pytest.mark.parametrize("N,d,V", SHAPES)
@pytest.mark.parametrize("reduction", ["mean", "none"])
def test_small_shapes(pingpong, N, d, V, reduction):
    inp = configs.make_inputs("tiny_track", N=N, d=d, V=V)
    ours = pu.run_ours(inp, reduction, keep_dlogits=True)
    ref = pu.run_oracle(inp, ours, reduction)
    print(pu.check_parity(ours, ref, reduction))


def test_ignored_rows_and_saturated_rows(pingpong):
    inp = configs.make_inputs("irregular", N=1500, d=256, V=3000)
    ours = pu.run_ours(inp, "mean", keep_dlogits=True)
    ref = pu.run_oracle(inp, ours, "mean")
    rep = pu.check_parity(ours, ref, "mean")
    assert rep["n_ignored"] > 0
    print(rep)


def test_agrees_with_the_default_kernel(monkeypatch):
    """lse and the losses come from the same accumulators summed in a different order; the stored dlogits are the same
    numbers with the same block exponents except where that order moves an exponent's floor: gradients to e4m3 precision."""
    inp = configs.make_inputs("limited_2p7b", N=2000, d=512, V=6000)
    a = pu.run_ours(inp, "none", keep_dlogits=True)
    monkeypatch.setenv("SCE_FWD_KERNEL", "pingpong")
    b = pu.run_ours(inp, "none", keep_dlogits=True)
    assert float((a["lse"] - b["lse"]).abs().max()) < 2e-6
    assert float((a["loss"] - b["loss"]).abs().max()) < 4e-6
    assert torch.equal(a["argmax"], b["argmax"])
    for k in ("dx", "dw"):
        assert pu.maxrel(b[k].float(), a[k].float()) < 5e-3, k


@pytest.mark.parametrize("beta_max", [14.0, 20.0])
def test_peaked_rows(pingpong, beta_max):
    """Rows the model is sure of: the target is the largest value of its block and stays out of its exponent."""
    N, d, V = 2048, 256, 4096
    inp = make_peaked(N, d, V, beta_max, shared=bool(beta_max > 15), seed=int(beta_max), ignore=0.05)
    go = torch.full((N,), 1.0 / N, device="cuda")
    ours = pu.run_ours(inp, "none", x_dtype=torch.float32, w_dtype=torch.float32, grad_output=go, keep_dlogits=True)
    ref = pu.run_oracle(inp, ours, "none", grad_output=go)
    rep = pu.check_parity(ours, ref, "none")
    sure = (ours["y"] != -1) & (torch.exp(-ref["losses"]) > 0.5)
    rr = per_row_rel(ours["dx"][sure], ref["dx"][sure])
    rep["sure_rows"], rep["row_rel_median"], rep["row_rel_max"] = int(sure.sum()), float(rr.median()), float(rr.max())
    print(rep)
    assert int(sure.sum()) > 100
    assert float(rr.median()) < 1e-2 and float(rr.max()) < 5e-2, rep


def test_multi_token_prediction(pingpong):
    from slowrun_amd.cuda_kernels import FusedSoftcappedCrossEntropy
    N, d, V = 1536, 256, 3000
    weights = [1.0, 0.7, 0.4, 0.2]
    inp = make_peaked(N, d, V, 16.0, shared=True, seed=5, ignore=0.03)
    inp.targets[200:260] = inp.targets[200]            # offsets of one row with the same target
    x = inp.x.cuda().requires_grad_(True)
    w = inp.w.cuda().requires_grad_(True)
    y = inp.targets.cuda()
    mw = torch.tensor(weights, device="cuda")
    go = torch.rand(N, generator=torch.Generator().manual_seed(3)).cuda() / N
    losses = FusedSoftcappedCrossEntropy.apply(x, y, mw, w, inp.x_s, inp.w_s, 0.75 / 448, 1.0, inp.cap)
    (losses * go).sum().backward()
    ref = eager.softcapped_ce_mtp(x.detach(), w.detach(), y, weights, inp.x_s, inp.w_s, cap=inp.cap, grad_output=go)
    assert float((losses.detach() - ref["loss"]).abs().max() / ref["loss"].abs().max()) < pu.LOSS_RTOL
    for name, got, want in (("dx", x.grad, ref["dx"]), ("dw", w.grad, ref["dw"])):
        mr, cs = pu.maxrel(got.float(), want), pu.cosine(got.float(), want)
        assert mr <= pu.GRAD_MAXREL and cs > pu.GRAD_COS, (name, mr, cs)


def test_tiny_track_shape_in_full(pingpong):
    inp = configs.make_inputs("tiny_track")
    ours = pu.run_ours(inp, "mean", keep_dlogits=True)
    ref = pu.run_oracle(inp, ours, "mean", row_chunk=4096)
    print(pu.check_parity(ours, ref, "mean"))
