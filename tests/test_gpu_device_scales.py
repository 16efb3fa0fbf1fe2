"""Scales that live on the device (0-dim tensors for x_s / w_s): nothing is read on the host, the kernels pick the
values up when they run.  The reference builds device scalars for its GEMMs from Python floats
(tiny/cuda_kernels.py:349-350,384-386); a trainer that rescales per step has them on the device to begin with.
torch divides a tensor by a tensor element by element (by a Python float it multiplies by the reciprocal), and so
does the quantiser here."""
import pytest
import torch

from oracle import eager
from slowrun_amd import configs
from tests import parity_util as pu

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_quantiser_with_a_device_scale_matches_torch_bit_for_bit(dtype):
    from slowrun_amd import cuda_kernels as ck
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(1 << 20, generator=g) * 3).to(dtype).cuda()
    for sv in (100 / 448, 0.0123, 0.761511070387704e-3):
        s = torch.tensor(sv, device="cuda", dtype=torch.float32)
        ours = ck.quantize_e4m3(x, s).view(torch.uint8)
        ref = x.div(s).to(torch.float8_e4m3fn).view(torch.uint8)          # tiny/cuda_kernels.py:340 with a tensor scale
        assert torch.equal(ours, ref), f"scale {sv}: {(ours != ref).sum().item()} bytes differ"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_amax_scale(dtype):
    from slowrun_amd import cuda_kernels as ck
    g = torch.Generator().manual_seed(2)
    t = (torch.randn(1000, 777, generator=g) * 5).to(dtype).cuda()
    s = ck.amax_scale(t)
    assert s.shape == () and s.dtype == torch.float32
    assert torch.equal(s.cpu(), t.abs().max().float().cpu() / 448.0)      # (divided on the CPU: there torch divides, on the GPU it multiplies by 1/448)
    t[5, 5] = float("nan")
    assert torch.isnan(ck.amax_scale(t))


@pytest.mark.parametrize("keep", [False, True])
def test_forward_backward_with_device_scales_against_the_oracle(keep):
    from slowrun_amd import cuda_kernels as ck
    inp = configs.make_inputs("irregular", N=1500, d=256, V=3000)
    x = inp.x.cuda().bfloat16()
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda()
    N, d = x.shape
    V = w.shape[1]
    xs, ws = ck.amax_scale(x), ck.amax_scale(w)
    out, saved, lse, argmax, n_valid = ck.ce_forward(x, w, y, xs, ws, inp.cap, "mean", want_argmax=True, keep_dlogits=keep)
    dx, dw = ck.ce_backward(saved, y, torch.ones((), device="cuda"), N, d, V, xs, ws, inp.cap, 1.0, "mean", torch.bfloat16,
                            torch.bfloat16, keep_dlogits=keep)
    ref = eager.softcapped_ce(x, w, y, xs, ws, cap=inp.cap, reduction="mean")       # torch divides by the tensors
    ours = dict(loss=out, lse=lse, argmax=argmax, n_valid=n_valid, dx=dx, dw=dw, x=x, w=w, y=y, x_s=xs, w_s=ws)
    print(pu.check_parity(ours, ref, "mean"))


def test_autograd_function_with_device_scales_in_a_hip_graph():
    """The trainer's call with tensor scales, amax pass included, captured once and replayed on new inputs: every
    replay must give the bits of the same calls issued directly (nothing was read on the host at capture time)."""
    from slowrun_amd import cuda_kernels as ck
    inp = configs.make_inputs("limited_2p7b", N=1200, d=256, V=2100)
    N, d, V = inp.shape
    x = inp.x.cuda().bfloat16()
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda()
    go = torch.ones((), device="cuda")

    def step():
        xs, ws = ck.amax_scale(x), ck.amax_scale(w)
        loss, saved, _lse, _am, _nv = ck.ce_forward(x, w, y, xs, ws, inp.cap, "mean", keep_dlogits=True)
        dx, dw = ck.ce_backward(saved, y, go, N, d, V, xs, ws, inp.cap, 1.0, "mean", torch.bfloat16, torch.bfloat16, keep_dlogits=True)
        return loss, dx, dw, xs

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    gen = torch.Generator().manual_seed(5)
    seen = set()
    for trial in range(4):
        x.copy_((inp.x * (1.0 + 0.7 * trial) + 0.05 * torch.randn(inp.x.shape, generator=gen)).bfloat16())     # the amax moves with it
        w.copy_((inp.w * (1.0 - 0.2 * trial)).bfloat16())
        y.copy_(torch.randint(0, V, (N,), generator=gen))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()
        torch.cuda.synchronize()
        for g_, e_, name in zip(got, want, ("loss", "dx", "dw", "x_s")):
            assert torch.equal(g_, e_), f"replay {trial}: {name} differs from the direct calls"
        assert torch.isfinite(got[0])
        seen.add(float(got[3]))
    assert len(seen) == 4                   # the scale did change from replay to replay


def test_trainer_call_with_tensor_scales():
    from slowrun_amd.cuda_kernels import FusedSoftcappedCrossEntropy
    inp = configs.make_inputs("tiny_track", N=640, d=128, V=1100)
    x = inp.x.cuda().bfloat16().requires_grad_(True)
    w = inp.w.cuda().bfloat16().requires_grad_(True)
    y = inp.targets.cuda()
    xs = torch.tensor(inp.x_s, device="cuda")
    ws = torch.tensor(inp.w_s, device="cuda")
    losses = FusedSoftcappedCrossEntropy.apply(x, y, None, w, xs, ws, 0.75 / 448, 1.0)
    losses.mean().backward()
    ref = eager.softcapped_ce(x.detach(), w.detach(), y, xs, ws, cap=15.0, reduction="none")
    assert float((losses.detach() - ref["loss"]).abs().max() / ref["loss"].abs().max()) < pu.LOSS_RTOL
    assert pu.cosine(x.grad.float(), ref["dx"]) > pu.GRAD_COS and pu.cosine(w.grad.float(), ref["dw"]) > pu.GRAD_COS
    assert pu.maxrel(x.grad.float(), ref["dx"]) <= pu.GRAD_MAXREL and pu.maxrel(w.grad.float(), ref["dw"]) <= pu.GRAD_MAXREL
