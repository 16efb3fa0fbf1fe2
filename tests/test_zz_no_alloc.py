"""sce_forward_noalloc (scratch in a static device array of the library) against sce_forward (scratch in the
caller's workspace), through the C ABI: the same kernels on the same inputs must give the same bits -- loss, per-row
losses, lse, argmax, counts, and through the saved state the gradients -- on two calls in a row that share the array, the second with
a smaller input, in both modes of the dlogits; sizes beyond the array are refused with a message."""
import pytest
import torch

from slowrun_amd import configs

pytestmark = pytest.mark.gpu


def _both(inp, reduction, keep):
    from slowrun_amd import cuda_kernels as ck
    x = inp.x.cuda().bfloat16()
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda()
    res = []
    for no_alloc in (False, True):
        out, saved, lse, argmax, n_valid = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, reduction, want_argmax=True,
                                                         keep_dlogits=keep, no_alloc=no_alloc)
        torch.cuda.synchronize()
        res.append((out, saved, lse, argmax, n_valid))
    return res, (x, w, y)


@pytest.mark.parametrize("keep", [False, True])
def test_no_alloc_forward_matches_forward_on_two_calls_in_a_row(keep):
    from slowrun_amd import cuda_kernels as ck
    from tests import parity_util as pu
    for (N, d, V), reduction in (((3000, 256, 5000), "mean"), ((700, 128, 1500), "none")):      # the second call is the smaller one
        inp = configs.make_inputs("irregular", N=N, d=d, V=V)
        (ref, got), (x, w, y) = _both(inp, reduction, keep)
        for name, a, b in zip(("loss", "saved", "lse", "argmax", "n_valid"), ref, got):
            if name != "saved":             # (its padding and unused regions are whatever the allocator left there)
                assert torch.equal(a, b), f"{name} differs at N={N} (keep_dlogits={keep})"
        # the state it saved -- quantised operands, row statistics, with keep_dlogits the dlogits -- drives a backward pass to the same bits
        go = torch.ones((), device="cuda") if reduction == "mean" else torch.full((N,), 1.0 / N, device="cuda")
        dx, dw = ck.ce_backward(got[1], y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, reduction, torch.bfloat16, torch.bfloat16,
                                keep_dlogits=keep)
        dx0, dw0 = ck.ce_backward(ref[1], y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, reduction, torch.bfloat16, torch.bfloat16,
                                  keep_dlogits=keep)
        assert torch.equal(dx, dx0) and torch.equal(dw, dw0)


def test_no_alloc_forward_refuses_what_does_not_fit():
    from slowrun_amd import cuda_kernels as ck
    N, d, V = 70000, 64, 4096                 # 70144 padded rows x 12 splits x 16 bytes > 8 MiB
    x = torch.zeros(N, d, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(d, V, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(N, dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="static scratch"):
        ck.ce_forward(x, w, y, 1.0, 1.0, 15.0, "mean", no_alloc=True)
    out, *_ = ck.ce_forward(x, w, y, 1.0, 1.0, 15.0, "mean")             # with a workspace the same call goes through
    assert abs(float(out) - float(torch.log(torch.tensor(float(V))))) < 1e-4
