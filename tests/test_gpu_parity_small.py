"""GPU parity of the HIP path against the oracle on small and ragged shapes,
through the C ABI (slowrun_amd.cuda_kernels -> libslowrun_ce.so)."""
import pytest
import torch

from slowrun_amd import configs
from tests import parity_util as pu

pytestmark = pytest.mark.gpu


def _small(name, N, d, V):
    return configs.make_inputs(name, N=N, d=d, V=V)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_quantize_matches_torch_cast_bit_exact(dtype):
    from slowrun_amd import cuda_kernels as ck
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(1 << 20, generator=g) * 3).to(dtype).cuda()
    x[:8] = torch.tensor([448., 449., 464., 465., 1e4, -1e4, 2.0 ** -10, 0.0], dtype=dtype)
    for s in (100 / 448, 1.6 / 448, 0.0123, 1.0):
        ours = ck.quantize_e4m3(x, s).view(torch.uint8)
        ref = x.div(s).to(torch.float8_e4m3fn).view(torch.uint8)      # tiny/cuda_kernels.py:340
        assert torch.equal(ours, ref), f"scale {s}: {(ours != ref).sum().item()} bytes differ"


def test_transpose_copy():
    from slowrun_amd import cuda_kernels as ck
    src = torch.randint(0, 255, (1000, 333), dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
    dst = torch.empty(333, 1000, dtype=torch.float8_e4m3fn, device="cuda")
    ck.transpose_copy(src, dst)
    assert torch.equal(dst.view(torch.uint8), src.view(torch.uint8).T.contiguous())


@pytest.mark.parametrize("N,d,V", [(256, 128, 256), (300, 128, 1000), (1000, 80, 777), (513, 272, 2049), (64, 16, 50304)])
@pytest.mark.parametrize("reduction", ["mean", "none"])
@pytest.mark.parametrize("keep", [False, True])
def test_small_shapes(N, d, V, reduction, keep):
    inp = _small("tiny_track", N, d, V)
    ours = pu.run_ours(inp, reduction, keep_dlogits=keep)
    ref = pu.run_oracle(inp, ours, reduction)
    print(pu.check_parity(ours, ref, reduction))


def test_small_fp32_inputs_and_ignored_rows():
    inp = _small("irregular", 700, 128, 1500)
    ours = pu.run_ours(inp, "mean", x_dtype=torch.float32, w_dtype=torch.float32)
    ref = pu.run_oracle(inp, ours, "mean")
    rep = pu.check_parity(ours, ref, "mean")
    assert rep["n_ignored"] > 0
    print(rep)


def test_small_panels_and_upstream_gradient():
    inp = _small("limited_2p7b", 1100, 256, 3000)
    go = torch.rand(1100, generator=torch.Generator().manual_seed(9)).cuda() * 2e-3
    ours = pu.run_ours(inp, "none", grad_output=go, panel_rows=256)
    ref = pu.run_oracle(inp, ours, "none", grad_output=go)
    print(pu.check_parity(ours, ref, "none"))
    ours2 = pu.run_ours(inp, "none", grad_output=go, panel_rows=0)
    assert pu.maxrel(ours2["dw"].float(), ours["dw"].float()) < 1e-2
    assert torch.equal(ours2["dx"], ours["dx"])


def test_all_rows_ignored():
    inp = _small("tiny_track", 300, 128, 512)
    inp.targets[:] = -1
    ours = pu.run_ours(inp, "mean")
    assert torch.isnan(ours["loss"])
    assert float(ours["dx"].float().abs().max()) == 0 and float(ours["dw"].float().abs().max()) == 0
    assert int(ours["n_valid"][0]) == 0


def test_out_of_range_targets_are_ignored_and_counted():
    inp = _small("tiny_track", 300, 128, 512)
    inp.targets[5] = 512
    inp.targets[7] = -7
    ours = pu.run_ours(inp, "none")
    assert int(ours["n_valid"][1]) == 2 and int(ours["n_valid"][0]) == 298
    assert float(ours["loss"][5]) == 0 and float(ours["loss"][7]) == 0
    assert float(ours["dx"][5].float().abs().max()) == 0


def test_autograd_function_signature():
    from slowrun_amd.cuda_kernels import CE_KERNEL_VOCAB_SIZE, FusedSoftcappedCrossEntropy
    assert CE_KERNEL_VOCAB_SIZE == 50304
    inp = _small("tiny_track", 512, 128, 1024)
    x = inp.x.cuda().bfloat16().requires_grad_(True)
    w = inp.w.cuda().bfloat16().requires_grad_(True)
    y = inp.targets.cuda()
    # the trainer's call (tiny/train.py:694-696) and reduction (tiny/train.py:1417-1419)
    losses = FusedSoftcappedCrossEntropy.apply(x, y, torch.tensor([1.0], device="cuda"), w, inp.x_s, inp.w_s, 0.75 / 448, 1.0)
    assert losses.shape == (512,)
    losses.mean().backward()
    assert x.grad.shape == x.shape and w.grad.shape == w.shape and w.grad.dtype == torch.bfloat16
    from oracle import eager
    ref = eager.softcapped_ce(x.detach(), w.detach(), y, inp.x_s, inp.w_s, cap=15.0, reduction="none")
    assert float((losses.detach() - ref["loss"]).abs().max() / ref["loss"].abs().max()) < 1e-3
    assert pu.cosine(x.grad.float(), ref["dx"]) > pu.GRAD_COS and pu.cosine(w.grad.float(), ref["dw"]) > pu.GRAD_COS


@pytest.mark.parametrize("weights", [[1.0], [1.0, 0.5, 0.25], [1.0, 0.5, 0.25, 0.125], [1.0, 0.0, 0.0]])
def test_multi_token_prediction(weights):
    """Per-row MTP losses and gradients against the oracle (tiny/cuda_kernels.py:226-301 semantics with the
    offsets that take no part left out of the gradient as well)."""
    from oracle import eager
    from slowrun_amd.cuda_kernels import FusedSoftcappedCrossEntropy
    inp = _small("irregular", 777, 128, 1300)        # has -1 targets, so some offsets drop out
    x = inp.x.cuda().bfloat16().requires_grad_(True)
    w = inp.w.cuda().bfloat16().requires_grad_(True)
    y = inp.targets.cuda()
    mw = torch.tensor(weights, device="cuda")
    go = torch.rand(777, generator=torch.Generator().manual_seed(3)).cuda() / 777
    losses = FusedSoftcappedCrossEntropy.apply(x, y, mw, w, inp.x_s, inp.w_s, 0.75 / 448, 1.0, inp.cap)   # trainer call
    (losses * go).sum().backward()
    ref = eager.softcapped_ce_mtp(x.detach(), w.detach(), y, weights, inp.x_s, inp.w_s, cap=inp.cap, grad_output=go)
    assert float((losses.detach() - ref["loss"]).abs().max() / ref["loss"].abs().max()) < pu.LOSS_RTOL
    for got, want in ((x.grad, ref["dx"]), (w.grad, ref["dw"])):
        assert pu.maxrel(got.float(), want) <= pu.GRAD_MAXREL and pu.cosine(got.float(), want) > pu.GRAD_COS
    if weights == [1.0, 0.0, 0.0]:
        plain = FusedSoftcappedCrossEntropy.apply(x.detach(), y, None, w.detach(), inp.x_s, inp.w_s, 0.75 / 448, 1.0, inp.cap)
        # the same up to the order of the fp32 sum over the columns (the targets of the zero-weight offsets take their
        # own way into the row sums)
        assert torch.allclose(plain, losses.detach(), rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("keep", [False, True])
@pytest.mark.parametrize("x_dtype", [torch.bfloat16, torch.float32])
def test_multi_token_prediction_through_both_dx_epilogues(keep, x_dtype):
    """Enough dX tiles in one panel (14 row tiles x 10 column tiles) for the staged epilogue that takes several
    offsets; with 256-row panels each tile's K loop is shared out and the finishing kernel applies the offsets: the two
    must give the same bf16 values, and both agree with the oracle."""
    from oracle import eager
    from slowrun_amd import cuda_kernels as ck
    N, d, V = 3400, 2560, 600
    weights = [1.0, 0.6, 0.3, 0.1]
    inp = _small("irregular", N, d, V)
    x = inp.x.cuda().to(x_dtype)
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda()
    mw = torch.tensor(weights, device="cuda")
    go = torch.rand(N, generator=torch.Generator().manual_seed(5)).cuda() / N
    out, saved, _lse, _am, _nv = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "none", mtp_weights=mw, keep_dlogits=keep)
    args = (saved, y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "none", x_dtype, torch.bfloat16)
    dx1, dw1 = ck.ce_backward(*args, mtp_weights=mw, keep_dlogits=keep)
    dx2, dw2 = ck.ce_backward(*args, mtp_weights=mw, keep_dlogits=keep, panel_rows=256)
    torch.cuda.synchronize()
    if x_dtype == torch.bfloat16:
        assert torch.equal(dx1, dx2)
    else:       # the shared-out K loop sums its fp32 parts in another order: visible in fp32 output
        assert pu.maxrel(dx1, dx2) < 1e-5
    ref = eager.softcapped_ce_mtp(x, w, y, weights, inp.x_s, inp.w_s, cap=inp.cap, grad_output=go)
    assert float((out - ref["loss"]).abs().max() / ref["loss"].abs().max()) < pu.LOSS_RTOL
    for got, want in ((dx1, ref["dx"]), (dw1, ref["dw"])):
        assert pu.maxrel(got.float(), want) <= pu.GRAD_MAXREL and pu.cosine(got.float(), want) > pu.GRAD_COS
    ign = y == -1
    assert int(ign.sum()) > 0


def test_traced_by_torch_compile():
    """The trainer wraps its model in torch.compile (tiny/train.py:1254): the loss head must trace without
    a graph break and give the eager result."""
    from slowrun_amd.cuda_kernels import FusedSoftcappedCrossEntropy
    inp = _small("tiny_track", 512, 128, 1024)
    x0 = inp.x.cuda().bfloat16()
    w0 = inp.w.cuda().bfloat16()
    y = inp.targets.cuda()
    mw = torch.tensor([1.0, 0.5], device="cuda")

    def head(x, w):
        h = x * 1.0
        return FusedSoftcappedCrossEntropy.apply(h, y, mw, w, inp.x_s, inp.w_s, 0.75 / 448, 1.0).mean()

    res = []
    for fn in (head, torch.compile(head, fullgraph=True, dynamic=False)):
        x = x0.clone().requires_grad_(True)
        w = w0.clone().requires_grad_(True)
        loss = fn(x, w)
        loss.backward()
        res.append((loss.detach(), x.grad, w.grad))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1]) and torch.equal(res[0][2], res[1][2])


def test_eval_head_with_vocabulary_slice():
    """tiny/train.py:741-743: logits sliced to the real vocabulary before softcap and cross entropy."""
    import torch.nn.functional as F
    from oracle import eager
    from slowrun_amd.cuda_kernels import softcapped_cross_entropy
    inp = _small("irregular", 600, 128, 1024)
    vocab = 1000
    inp.targets[inp.targets >= vocab] = 3
    x = inp.x.cuda().bfloat16().reshape(3, 200, 128)
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda().reshape(3, 200)
    xq = eager.dequantize(eager.quantize_e4m3(x.reshape(-1, 128), inp.x_s), inp.x_s)
    wq = eager.dequantize(eager.quantize_e4m3(w, inp.w_s), inp.w_s)
    logits = (xq @ wq)[..., :vocab].float()
    logits = inp.cap * torch.tanh(logits / inp.cap)
    for red in ("mean", "none"):
        ref = F.cross_entropy(logits, y.reshape(-1), ignore_index=-1, reduction=red)
        got = softcapped_cross_entropy(x, w, y, inp.x_s, inp.w_s, cap=inp.cap, vocab_size=vocab, reduction=red)
        assert got.shape == (() if red == "mean" else (3, 200))
        assert float((got.reshape(-1) - ref.reshape(-1)).abs().max() / ref.abs().max()) < pu.LOSS_RTOL


def test_target_probability_of_the_ensemble_evaluation():
    """unlimited/train.py:1063-1069: p(target) = exp(logit[target] - logsumexp(logits)) from the full logits; here from
    the per-row losses, with bf16 operands as the reference's evaluation has them under autocast."""
    from slowrun_amd.cuda_kernels import target_probability
    inp = _small("irregular", 600, 128, 1024)
    x = inp.x.cuda().bfloat16().reshape(3, 200, 128)
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda().reshape(3, 200)
    logits = (x.reshape(-1, 128) @ w).float()                      # bf16 result of the bf16 matmul, then fp32
    logits = inp.cap * torch.tanh(logits / inp.cap)
    valid = y.reshape(-1) != -1
    logit_gt = logits.gather(1, y.reshape(-1).clamp(min=0).unsqueeze(1)).squeeze(1)
    ref = torch.exp(logit_gt - torch.logsumexp(logits, dim=-1))
    got = target_probability(x, w, y, cap=inp.cap, operand_dtype=torch.bfloat16)
    assert got.shape == (3, 200)
    assert float((got.reshape(-1)[valid] - ref[valid]).abs().max() / ref[valid].max()) < pu.LOSS_RTOL
    assert int((~valid).sum()) > 0 and float(got.reshape(-1)[~valid].abs().max()) == 0.0
    # e4m3 operands: against the oracle's per-row losses
    from oracle import eager
    got8 = target_probability(x, w, y, inp.x_s, inp.w_s, cap=inp.cap)
    ref8 = eager.softcapped_ce(x.reshape(-1, 128), w, y.reshape(-1), inp.x_s, inp.w_s, cap=inp.cap, reduction="none", want_grads=False)
    want = torch.exp(-ref8["loss"])
    assert float((got8.reshape(-1)[valid] - want[valid]).abs().max() / want[valid].max()) < pu.LOSS_RTOL


def test_vocabulary_slice_backward_and_weight_cache():
    from oracle import eager
    from slowrun_amd import cuda_kernels as ck
    inp = _small("tiny_track", 520, 128, 1024)
    vocab = 900
    inp.targets[inp.targets >= vocab] = 7
    x = inp.x.cuda().bfloat16()
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda()
    # oracle: zero weight columns do not reproduce a slice (they still enter the softmax), so slice W itself
    ref = eager.softcapped_ce(x, w[:, :vocab].contiguous(), y, inp.x_s, inp.w_s, cap=inp.cap, reduction="mean")
    cache = ck.WeightCache()
    go = torch.ones((), device="cuda")
    for rep in range(2):                      # second pass reuses the cached quantised W
        loss, saved, _lse, _am, _nv = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "mean", vocab_size=vocab,
                                                    weight_cache=cache)
        dx, dw = ck.ce_backward(saved, y, go, 520, 128, 1024, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16,
                                torch.bfloat16, vocab_size=vocab, weight_cache=cache)
        assert abs(float(loss) - float(ref["loss"])) / float(ref["loss"]) < pu.LOSS_RTOL
        assert pu.cosine(dx.float(), ref["dx"]) > pu.GRAD_COS and pu.maxrel(dx.float(), ref["dx"]) < pu.GRAD_MAXREL
        assert pu.cosine(dw[:, :vocab].float(), ref["dw"]) > pu.GRAD_COS
        assert float(dw[:, vocab:].float().abs().max()) == 0.0
        if rep == 0:
            first = (loss.clone(), dx.clone(), dw.clone())
    assert torch.equal(first[0], loss) and torch.equal(first[1], dx) and torch.equal(first[2], dw)
    # a changed weight invalidates the cache
    w2 = w.clone()
    w2[:, :10] *= 0.5
    loss2, *_ = ck.ce_forward(x, w2, y, inp.x_s, inp.w_s, inp.cap, "mean", vocab_size=vocab, weight_cache=cache)
    loss2_nocache, *_ = ck.ce_forward(x, w2, y, inp.x_s, inp.w_s, inp.cap, "mean", vocab_size=vocab)
    assert torch.equal(loss2, loss2_nocache) and not torch.equal(loss2, loss)
    w2.mul_(0.5)                                  # in-place update bumps the version counter
    loss3, *_ = ck.ce_forward(x, w2, y, inp.x_s, inp.w_s, inp.cap, "mean", vocab_size=vocab, weight_cache=cache)
    loss3_nocache, *_ = ck.ce_forward(x, w2, y, inp.x_s, inp.w_s, inp.cap, "mean", vocab_size=vocab)
    assert torch.equal(loss3, loss3_nocache)
    # a write through .data is invisible to the version counter (tiny/train.py:1586 broadcasts parameters that way):
    # the cache has to be told
    w2.data.mul_(2.0)
    gen = cache.generation
    stale, *_ = ck.ce_forward(x, w2, y, inp.x_s, inp.w_s, inp.cap, "mean", vocab_size=vocab, weight_cache=cache)
    assert torch.equal(stale, loss3) and cache.generation == gen
    cache.invalidate()
    loss4, saved4, *_ = ck.ce_forward(x, w2, y, inp.x_s, inp.w_s, inp.cap, "mean", vocab_size=vocab, weight_cache=cache)
    loss4_nocache, *_ = ck.ce_forward(x, w2, y, inp.x_s, inp.w_s, inp.cap, "mean", vocab_size=vocab)
    assert torch.equal(loss4, loss4_nocache) and cache.generation == gen + 1
    # a backward that belongs to an older fill of the cache is refused
    with pytest.raises(RuntimeError, match="refilled"):
        ck.ce_backward(saved4, y, go, 520, 128, 1024, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16, torch.bfloat16,
                       vocab_size=vocab, weight_cache=cache, cache_generation=gen)


def test_minimum_workspace_and_strided_rows():
    """Smallest allowed backward workspace: 256-row panels, a single fp32 dW buffer that later launches read,
    add to and rewrite.  Also feeds X and W as row-strided views (row stride > row length)."""
    from slowrun_amd import _lib
    from slowrun_amd import cuda_kernels as ck
    inp = _small("limited_2p7b", 1300, 256, 2100)
    xbig = torch.zeros(1300, 300, dtype=torch.bfloat16, device="cuda")
    wbig = torch.zeros(256, 2200, dtype=torch.bfloat16, device="cuda")
    xbig[:, :256] = inp.x.cuda().bfloat16()
    wbig[:, :2100] = inp.w.cuda().bfloat16()
    x, w = xbig[:, :256], wbig[:, :2100]              # stride(0) = 300 / 2200, stride(1) = 1
    y = inp.targets.cuda()
    sz = _lib.sizes_for(1300, 256, 2100)
    loss, saved, lse, _am, _nv = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "mean")
    go = torch.ones((), device="cuda")
    dx_min, dw_min = ck.ce_backward(saved, y, go, 1300, 256, 2100, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16,
                                    torch.float32, workspace_bytes=sz.bwd_workspace_min_bytes)
    ours = dict(loss=loss, lse=lse, argmax=None, n_valid=_nv, dx=dx_min, dw=dw_min, x=x.contiguous(), w=w.contiguous(), y=y,
                x_s=inp.x_s, w_s=inp.w_s)
    ref = pu.run_oracle(inp, ours, "mean")
    print(pu.check_parity(ours, ref, "mean", check_argmax=False))
    dx_def, dw_def = ck.ce_backward(saved, y, go, 1300, 256, 2100, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16,
                                    torch.float32)
    assert torch.equal(dx_def, dx_min)
    assert pu.maxrel(dw_def, dw_min) < 1e-4          # same terms, different order of the fp32 sums
    with pytest.raises(RuntimeError, match="workspace too small"):
        ck.ce_backward(saved, y, go, 1300, 256, 2100, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16, torch.float32,
                       workspace_bytes=sz.bwd_workspace_min_bytes - 4096)


def test_fixed_scales_of_the_trainer_and_overflow_to_nan():
    """The trainer's fixed scales (tiny/train.py:188-189).  A value that overflows e4m3 becomes NaN in torch's
    cast and poisons that row's loss in the eager path; the fused path must do the same, not saturate."""
    from oracle import eager
    inp = _small("tiny_track", 300, 128, 700)
    x_s, w_s = 100 / 448, 1.6 / 448
    inp.x_s, inp.w_s = x_s, w_s
    ours = pu.run_ours(inp, "none")
    ref = pu.run_oracle(inp, ours, "none")
    print(pu.check_parity(ours, ref, "none"))
    inp.x[17, 5] = 150.0                              # 150 / x_s = 672 > 464 -> NaN code
    ours = pu.run_ours(inp, "none")
    ref = eager.softcapped_ce(ours["x"], ours["w"], ours["y"], x_s, w_s, cap=inp.cap, reduction="none", want_grads=False)
    assert torch.isnan(ref["loss"][17]) and torch.isnan(ours["loss"][17])
    ok = torch.ones(300, dtype=torch.bool, device="cuda")
    ok[17] = False
    assert float((ours["loss"][ok] - ref["loss"][ok]).abs().max()) < 1e-3


def test_frequent_target_segments_are_chunked():
    """One target shared by 3000 rows (its one-hot part of dW is summed in twelve chunks), one by 70 rows and one by
    exactly 16 (a single chunk each), one by 15 (one short of a chunk of its own) and the rest spread out (summed in
    the final kernel)."""
    inp = _small("tiny_track", 4096, 128, 512)
    inp.targets[:3000] = 7
    inp.targets[3000:3070] = 11
    others = inp.targets[3070:].clone()
    others[(others == 13) | (others == 17)] = 19
    inp.targets[3070:] = others
    inp.targets[3070:3086] = 13
    inp.targets[3086:3101] = 17
    ours = pu.run_ours(inp, "mean")
    ref = pu.run_oracle(inp, ours, "mean")
    print(pu.check_parity(ours, ref, "mean"))


def test_dx_panel_with_few_tiles_is_k_split():
    """512 rows x d = 256 is two dX tiles: each tile's K loop (V) is shared by several workgroups."""
    inp = _small("limited_2p7b", 512, 256, 8192)
    ours = pu.run_ours(inp, "none", x_dtype=torch.float32)
    ref = pu.run_oracle(inp, ours, "none")
    print(pu.check_parity(ours, ref, "none"))


def test_captured_in_a_hip_graph_and_replayed():
    """Every launch of forward and backward goes to the caller's stream and nothing synchronises, so the
    pair can be captured once and replayed on new contents of the same buffers (tiny/train.py:1254 compiles
    the model; a trainer that captures its step needs this).  Each replay is compared bit for bit with
    the same calls issued directly."""
    from slowrun_amd import cuda_kernels as ck
    inp = _small("limited_2p7b", 1500, 256, 2100)
    N, d, V = inp.shape
    x = inp.x.cuda().bfloat16()
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda()
    go = torch.ones((), device="cuda")

    def step():
        loss, saved, _lse, _am, _nv = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "mean")
        dx, dw = ck.ce_backward(saved, y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16, torch.bfloat16)
        return loss, dx, dw

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    gen = torch.Generator().manual_seed(21)
    for trial in range(4):
        amax = float(inp.x.abs().max())            # the scale x_s was taken from this: stay inside e4m3's range
        x.copy_((inp.x * (1.0 - 0.1 * trial) + 0.05 * torch.randn(inp.x.shape, generator=gen)).clamp(-amax, amax).bfloat16())
        y.copy_(torch.randint(0, V, (N,), generator=gen))
        if trial == 2:
            y[::7] = -1
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = step()
        torch.cuda.synchronize()
        for g, e, name in zip(got, want, ("loss", "dx", "dw")):
            assert torch.equal(g, e), f"replay {trial}: {name} differs from the direct calls"
        assert torch.isfinite(got[0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_final_norm_fused_into_the_head(dtype):
    """tiny/train.py:734 then :682-696: x = F.rms_norm(h, (d,)) feeds the head.  With the norm inside the quantiser
    the result must match the oracle (norm restated in fp32, head as everywhere else) and the unfused pair
    torch rms_norm -> FusedSoftcappedCrossEntropy on the same kernels."""
    import torch.nn.functional as F
    from oracle import eager
    from slowrun_amd.cuda_kernels import FusedNormSoftcappedCrossEntropy, FusedSoftcappedCrossEntropy
    inp = _small("irregular", 700, 256, 1500)
    N, d, V = inp.shape
    gen = torch.Generator().manual_seed(3)
    h_cpu = (inp.x * (0.5 + 2.5 * torch.rand(N, 1, generator=gen))).to(dtype)
    w_cpu = inp.w.to(dtype)
    x_ref, _ = eager.rms_norm(h_cpu)
    x_s = float(x_ref.float().abs().max()) / 448.0
    assert int((inp.targets == -1).sum()) > 0
    ref = eager.norm_softcapped_ce(h_cpu, w_cpu, inp.targets, x_s, inp.w_s, inp.cap, "mean")
    y = inp.targets.cuda()
    res = []
    for fused in (True, False):
        h = h_cpu.cuda().requires_grad_(True)
        w = w_cpu.cuda().requires_grad_(True)
        if fused:
            loss = FusedNormSoftcappedCrossEntropy.apply(h, y, None, w, x_s, inp.w_s, 0.0, 1.0, inp.cap, "mean")
        else:
            loss = FusedSoftcappedCrossEntropy.apply(F.rms_norm(h, (d,)), y, None, w, x_s, inp.w_s, 0.0, 1.0, inp.cap, "mean")
        loss.backward()
        res.append((loss.detach().cpu(), h.grad.float().cpu(), w.grad.float().cpu()))
    (loss, dh, dw), (loss_u, dh_u, dw_u) = res
    assert abs(float(loss) - float(ref["loss"])) <= 1e-3 * abs(float(ref["loss"]))
    for name, got, want in (("dh", dh, ref["dx"].float()), ("dw", dw, ref["dw"].float())):
        mr, cs = pu.maxrel(got, want), pu.cosine(got, want)
        print(name, mr, cs)
        assert mr <= 2e-2 and cs > 0.9995, (name, mr, cs)
    ignored = inp.targets == -1
    assert float(dh[ignored].abs().max()) == 0.0
    # torch's GPU rms_norm sums the squares in another order: in fp32 the last bit may differ, in bf16 a few
    # elements may round to the neighbouring value
    x_torch = F.rms_norm(h_cpu.cuda(), (d,)).cpu()
    if dtype == torch.float32:
        assert pu.maxrel(x_torch, x_ref) < 1e-6
    else:
        assert float((x_torch != x_ref).float().mean()) < 1e-3
    assert abs(float(loss) - float(loss_u)) <= 1e-5 * abs(float(loss_u))
    assert pu.maxrel(dh, dh_u) < 1e-2 and pu.maxrel(dw, dw_u) < 1e-2


def _random_shapes(seed, count):
    gen = torch.Generator().manual_seed(seed)
    shapes = []
    for _ in range(count):
        N = int(torch.randint(1, 2200, (1,), generator=gen))
        d = 16 * int(torch.randint(1, 40, (1,), generator=gen))
        V = int(torch.randint(2, 4000, (1,), generator=gen))
        shapes.append((N, d, V))
    return shapes


@pytest.mark.parametrize("N,d,V", [(1, 16, 2), (2, 16, 257), (255, 32, 255), (257, 48, 513)] + _random_shapes(1234, 10))
@pytest.mark.parametrize("keep", [False, True])
def test_ragged_and_tiny_shapes(N, d, V, keep):
    """Sizes on both sides of every tile boundary, down to one row, 16 hidden units and two columns: ignored rows
    included, panels of the smallest size and of the default size must agree with the oracle and with each other."""
    inp = _small("irregular", N, d, V)
    reduction = "none" if (N + d + V) % 2 else "mean"
    ours = pu.run_ours(inp, reduction, keep_dlogits=keep)
    ref = pu.run_oracle(inp, ours, reduction)
    # The stated gradient tolerance is for sums over many rows and columns.  The part of dlogits that is not the
    # one-hot term passes through e4m3 (three mantissa bits: steps of up to 6.25 %, the reference's e5m2 has twice
    # that); with a handful of rows or columns nothing averages out and a single rounding shows in full.
    tiny = N < 64 or V < 64
    rep = pu.check_parity(ours, ref, reduction, grad_maxrel=7e-2 if tiny else pu.GRAD_MAXREL,
                          grad_cos=0.999 if tiny else pu.GRAD_COS)
    small = pu.run_ours(inp, reduction, panel_rows=256, keep_dlogits=keep)
    assert torch.equal(small["dx"], ours["dx"])
    assert pu.maxrel(small["dw"].float(), ours["dw"].float()) < 1e-2
    print(N, d, V, reduction, rep)


@pytest.mark.parametrize("V", [1019, 900, 257])
@pytest.mark.parametrize("keep", [False, True])
def test_negative_logits_beside_columns_that_do_not_exist(V, keep):
    """Every logit below zero, in a vocabulary that ends inside a tile (inside a group of 32 columns, inside the second
    128-column half, one column into a tile): the columns a tile has beyond the vocabulary come out of the zero padding
    of W as logit 0, above every real one -- they must win neither the argmax nor a block's exponent, and add nothing
    to the row sums."""
    inp = _small("irregular", 300, 64, V)
    inp.x = inp.x.abs()
    inp.w = -inp.w.abs()
    ours = pu.run_ours(inp, "mean", keep_dlogits=keep)
    ref = pu.run_oracle(inp, ours, "mean")
    assert int(ours["argmax"].max()) < V
    print(V, keep, pu.check_parity(ours, ref, "mean"))


@pytest.mark.parametrize("N,d,V,keep,reduction", [(3518, 560, 9364, True, "none"), (4216, 832, 131, True, "mean"), (5549, 576, 133, False, "mean"),
                                                  (3183, 560, 290, True, "none"), (1267, 544, 8807, False, "none")])
def test_saturating_rows_with_an_unlucky_sample(N, d, V, keep, reduction):
    """Shapes (found by random search) in which one of the workload's few rows with 50-fold activations -- logits that
    saturate the cap -- has a group of 16 sampled columns without a positive one: taken at its word, the sample makes
    the row's level 2^-40, and with that boost the row sets the exponent of every block it is in; the 31 rows that
    share those blocks then lose their mantissa bits (dX off by 3 to 14 % of the largest entry).  The boost is limited."""
    inp = _small("irregular", N, d, V)
    ours = pu.run_ours(inp, reduction, keep_dlogits=keep)
    ref = pu.run_oracle(inp, ours, reduction)
    print(N, d, V, keep, reduction, pu.check_parity(ours, ref, reduction))


def test_fused_norm_with_multi_token_prediction_and_eval_head():
    """The fused norm composes with the other options: multi-token prediction in training, the vocabulary slice in
    evaluation.  Reference: the same calls on torch's own rms_norm output (bit-identical to the fused norm for bf16)."""
    import torch.nn.functional as F
    from slowrun_amd.cuda_kernels import (FusedNormSoftcappedCrossEntropy, FusedSoftcappedCrossEntropy,
                                          softcapped_cross_entropy)
    inp = _small("tiny_track", 900, 128, 1300)
    N, d, V = inp.shape
    gen = torch.Generator().manual_seed(11)
    h0 = (inp.x * (0.3 + 3.0 * torch.rand(N, 1, generator=gen))).bfloat16().cuda()
    w0 = inp.w.bfloat16().cuda()
    y = inp.targets.cuda()
    y[::9] = -1
    x_s = float(F.rms_norm(h0, (d,)).float().abs().max()) / 448.0
    mw = torch.tensor([1.0, 0.6, 0.3], device="cuda")
    res = []
    for fused in (True, False):
        h = h0.clone().requires_grad_(True)
        w = w0.clone().requires_grad_(True)
        if fused:
            losses = FusedNormSoftcappedCrossEntropy.apply(h, y, mw, w, x_s, inp.w_s, 0.0, 1.0)
        else:
            losses = FusedSoftcappedCrossEntropy.apply(F.rms_norm(h, (d,)), y, mw, w, x_s, inp.w_s, 0.0, 1.0)
        losses.mean().backward()
        res.append((losses.detach(), h.grad, w.grad))
    assert torch.equal(res[0][0], res[1][0])                  # same fp8 bytes in, same kernels: same losses
    assert torch.equal(res[0][2], res[1][2])                  # and the same dW
    assert pu.maxrel(res[0][1].float(), res[1][1].float()) < 1e-2 and pu.cosine(res[0][1].float(), res[1][1].float()) > 0.99999
    ev_fused = softcapped_cross_entropy(h0, w0, y, x_s, inp.w_s, vocab_size=1250, reduction="none",
                                        norm_eps=torch.finfo(torch.float32).eps)
    ev_plain = softcapped_cross_entropy(F.rms_norm(h0, (d,)), w0, y, x_s, inp.w_s, vocab_size=1250, reduction="none")
    assert torch.equal(ev_fused, ev_plain)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_eval_head_with_bf16_operands(dtype):
    """The reference evaluates with a bf16 matmul (CastedLinearT under autocast, tiny/train.py:496-497) whose bf16 logits
    are sliced to the vocabulary, softcapped and fed to F.cross_entropy in fp32 (tiny/train.py:741-743).  With
    operand_dtype=torch.bfloat16 the fused head computes that arithmetic: same operands, fp32 accumulation, logits
    rounded to bf16.  The two GEMMs add in different orders, so a logit may land on the neighbouring bf16 value (one
    part in 256 of it) now and then; the losses are compared at the tolerance stated for the loss."""
    import torch.nn.functional as F
    from slowrun_amd.cuda_kernels import softcapped_cross_entropy
    inp = _small("irregular", 1100, 256, 2300)
    vocab = 2250
    inp.targets[inp.targets >= vocab] = 3
    x = inp.x.cuda().to(dtype).reshape(2, 550, 256)
    w = inp.w.cuda().to(dtype)
    y = inp.targets.cuda().reshape(2, 550)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        logits = (x @ w.type_as(x))                                   # CastedLinearT.forward
    assert logits.dtype == torch.bfloat16
    logits = logits[..., :vocab].float()
    logits = inp.cap * torch.tanh(logits / inp.cap)
    for red in ("mean", "none"):
        ref = F.cross_entropy(logits.view(-1, vocab), y.reshape(-1), ignore_index=-1, reduction=red)
        got = softcapped_cross_entropy(x, w, y, cap=inp.cap, vocab_size=vocab, reduction=red, operand_dtype=torch.bfloat16)
        assert got.shape == (() if red == "mean" else (2, 550))
        err = float((got.reshape(-1) - ref.reshape(-1)).abs().max() / ref.abs().max())
        print(dtype, red, "rel err", err)
        assert err < pu.LOSS_RTOL if red == "mean" else err < 1e-2
    # the e4m3 path on the same data differs from the bf16 one by more than that: the two are not the same arithmetic
    fp8 = softcapped_cross_entropy(x, w, y, inp.x_s, inp.w_s, cap=inp.cap, vocab_size=vocab, reduction="none")
    bf = softcapped_cross_entropy(x, w, y, cap=inp.cap, vocab_size=vocab, reduction="none", operand_dtype=torch.bfloat16)
    assert float((fp8 - bf).abs().max()) > 1e-3


def test_bf16_operands_are_forward_only():
    from slowrun_amd import cuda_kernels as ck
    inp = _small("tiny_track", 300, 128, 600)
    x = inp.x.cuda().bfloat16()
    w = inp.w.cuda().bfloat16()
    y = inp.targets.cuda()
    loss, saved, *_ = ck.ce_forward(x, w, y, 1.0, 1.0, inp.cap, "mean", operand_dtype=torch.bfloat16)
    assert torch.isfinite(loss)
    with pytest.raises(ValueError, match="forward-only"):
        ck.ce_forward(x, w, y, 1.0, 1.0, inp.cap, "mean", operand_dtype=torch.bfloat16, keep_dlogits=True)


@pytest.mark.parametrize("N,d,V", [(2048, 512, 6000), (1024, 1024, 50304), (700, 272, 2049)])
def test_dw_with_and_without_the_k_split_last_round(N, d, V):
    """With room in the workspace a last round of dW tiles that is far from full is shared out along K (here: all of
    the tiles, there being fewer than CUs); without it every tile has one workgroup.  Same sums, in a different order."""
    from slowrun_amd import _lib, cuda_kernels as ck
    inp = _small("tiny_track", N, d, V)
    x, w, y = inp.x.cuda(), inp.w.cuda(), inp.targets.cuda()
    sz = _lib.sizes_for(N, d, V)
    out, saved, lse, _, _ = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "mean", keep_dlogits=True)
    go = torch.ones((), device="cuda")
    args = (saved, y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.float32, torch.float32)
    dx1, dw1 = ck.ce_backward(*args, keep_dlogits=True)
    # the same workspace without the room for the partial tiles: they lie at its end, one 256 x 256 fp32 tile for
    # each of the 256 workgroups and one more for each tile of the shared-out round
    tiles = -(-d // 256) * -(-V // 256)
    small = sz.bwd_workspace_kept_bytes - (256 + tiles % 256) * 256 * 256 * 4
    dx2, dw2 = ck.ce_backward(*args, keep_dlogits=True, workspace_bytes=small)
    torch.cuda.synchronize()
    assert torch.equal(dx1, dx2)
    assert pu.maxrel(dw1, dw2) < 2e-6


@pytest.mark.parametrize("keep", [False, True])
def test_more_rows_than_one_dw_launch_takes(keep):
    """A dW launch takes at most 131072 rows (its K loop): with more rows there are several launches, each with an fp32
    partial of its own, summed in a fixed order at the end; dX goes panel by panel as always."""
    N, d, V = 140000, 64, 600
    inp = _small("irregular", N, d, V)
    ours = pu.run_ours(inp, "mean", keep_dlogits=keep)
    ref = pu.run_oracle(inp, ours, "mean", row_chunk=16384)
    rep = pu.check_parity(ours, ref, "mean")
    assert rep["n_ignored"] > 0
    print(rep)


@pytest.mark.parametrize("keep", [False, True])
def test_largest_vocabulary(keep):
    """V = 524288 is the most the dX kernel takes (the block exponents of a tile's K loop, one per 128 columns, fill the
    LDS left beside the two K slots); one column beyond it is refused (tests/test_abi.py)."""
    N, d, V = 300, 64, 524288
    inp = _small("large_vocab", N, d, V)
    ours = pu.run_ours(inp, "mean", keep_dlogits=keep)
    ref = pu.run_oracle(inp, ours, "mean", row_chunk=64)
    print(pu.check_parity(ours, ref, "mean"))


@pytest.mark.parametrize("keep", [False, True])
def test_wide_hidden_size(keep):
    """d = 8208: a forward K loop of 66 blocks, 33 column tiles of dX per row tile, and a last tile of 16 columns."""
    N, d, V = 600, 8208, 1500
    inp = _small("limited_2p7b", N, d, V)
    ours = pu.run_ours(inp, "none", keep_dlogits=keep)
    ref = pu.run_oracle(inp, ours, "none")
    print(pu.check_parity(ours, ref, "none"))


@pytest.mark.parametrize("cap", [1.0, 5.0, 40.0])
@pytest.mark.parametrize("keep", [False, True])
def test_softcap_range(cap, keep):
    """The two ends of the allowed softcap and one between, on inputs with rows that saturate it: at cap = 40 the
    dlogits span e^-80 .. 1 (block exponents down to 2^-115), at cap = 1 every logit is within one unit of every other."""
    inp = _small("irregular", 700, 128, 2500)
    inp.cap = cap
    ours = pu.run_ours(inp, "mean", keep_dlogits=keep)
    ref = pu.run_oracle(inp, ours, "mean")
    rep = pu.check_parity(ours, ref, "mean")
    assert rep["n_ignored"] > 0
    print(rep)


@pytest.mark.parametrize("keep", [True, False])
@pytest.mark.parametrize("n_predict", [1, 3, 4])
@pytest.mark.parametrize("shape", [(700, 272, 2049), (513, 64, 300), (256, 128, 1000), (1031, 528, 5000)])
def test_target_logits_ahead_of_the_forward_kernel(shape, n_predict, keep):
    """An fp8 forward pass gets its target logits from a tile of gathered rows of W_q^T, computed before
    the forward kernel (which then never looks for a target in its accumulators), or -- for a W_q^T beyond the gather's
    32-bit offsets -- from the forward kernel's own accumulators.  sce_test_set_gather_limit forces the second way at a
    size a test can afford.  The argmax of the two ways is the same; the row sums take the target's term in at a
    different place (lse within 2 ulp, the losses with it), and the gradients agree up to the rounding of the
    dlogits (the blocks' exponents are found differently).  A forward pass that emits nothing does the same sums either
    way, and the backward pass that follows it is the same code: everything is equal bit for bit."""
    from slowrun_amd import _lib, cuda_kernels as ck
    N, d, V = shape
    g = torch.Generator().manual_seed(N + n_predict)
    from tests.test_gpu_parity_peaked import make_peaked
    inp = make_peaked(N, d, V, 12.0, shared=True, seed=N, ignore=0.1)
    x, w, y = inp.x.cuda(), inp.w.cuda(), inp.targets.cuda().clone()
    y[5:9] = y[5]                                  # offsets of one row with the same target
    y[N - 2] = -1
    mw = torch.rand(n_predict, generator=g).cuda() + 0.1 if n_predict > 1 else None
    go = (torch.rand(N, generator=g) / N).cuda()
    res = []
    lib = _lib.lib()
    try:
        for limit in (0, 1):
            lib.sce_test_set_gather_limit(limit)
            out, saved, lse, am, nv = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "none", mtp_weights=mw, keep_dlogits=keep, want_argmax=True)
            dx, dw = ck.ce_backward(saved, y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "none", torch.float32, torch.float32,
                                    mtp_weights=mw, keep_dlogits=keep)
            torch.cuda.synchronize()
            res.append((out.clone(), lse.clone(), am.clone(), nv.clone(), dx.clone(), dw.clone()))
    finally:
        lib.sce_test_set_gather_limit(0)
    a, b = res
    if not keep:
        assert all(torch.equal(u, v) for u, v in zip(a, b))
        return
    assert torch.equal(a[2], b[2]) and torch.equal(a[3], b[3])
    assert float((a[1] - b[1]).abs().max()) <= 4e-6 * float(b[1].abs().max().clamp_min(1.0))
    assert float((a[0] - b[0]).abs().max()) <= 2e-5
    for name, u, v in (("dx", a[4], b[4]), ("dw", a[5], b[5])):
        mr, cs = pu.maxrel(u, v), pu.cosine(u, v)
        assert mr <= pu.GRAD_MAXREL and cs > pu.GRAD_COS, (name, mr, cs)


@pytest.mark.parametrize("keep", [True, False])
@pytest.mark.parametrize("n_predict", [1, 3])
def test_head_that_starts_at_zero(keep, n_predict):
    """All logits are equal (W = 0, as a zero-initialised lm_head has it at the first step; here also a W with a few
    repeated columns): the target is then not the only one of a lane's values with its value, and the kernels that know
    their targets by value must not take the others for it."""
    from slowrun_amd import cuda_kernels as ck
    from oracle import eager
    N, d, V = 600, 128, 1500
    g = torch.Generator().manual_seed(11)
    x = torch.randn(N, d, generator=g).cuda()
    y = torch.randint(0, V, (N,), generator=g).cuda()
    y[7] = -1
    mw = torch.tensor([1.0, 0.5, 0.25][:n_predict]).cuda() if n_predict > 1 else None
    go = (torch.rand(N, generator=g) / N).cuda()
    x_s, w_s = float(x.abs().max()) / 448.0, 1.6 / 448.0
    for w in (torch.zeros(d, V).cuda(), (torch.randn(d, 1, generator=g) * d ** -0.5).expand(d, V).contiguous().cuda()):
        out, saved, lse, am, nv = ck.ce_forward(x, w, y, x_s, w_s, 15.0, "none", mtp_weights=mw, keep_dlogits=keep)
        dx, dw = ck.ce_backward(saved, y, go, N, d, V, x_s, w_s, 15.0, 1.0, "none", torch.float32, torch.float32, mtp_weights=mw,
                                keep_dlogits=keep)
        torch.cuda.synchronize()
        assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(dx).all()) and bool(torch.isfinite(dw).all())
        ref = eager.softcapped_ce_mtp(x, w, y, [1.0, 0.5, 0.25][:n_predict], x_s, w_s, cap=15.0, grad_output=go)
        assert float((out - ref["loss"]).abs().max() / ref["loss"].abs().max()) < pu.LOSS_RTOL
        # dX is zero in exact arithmetic (every column of W is the same vector w: sum_v p_v w - w = 0); what comes out is the
        # rounding of the dlogits, all of a row's alike here, against the scale g w of its two terms
        scale = float(go.max()) * float(w.abs().max()) * (float(mw.sum()) if mw is not None else 1.0)
        assert float(dx.abs().max()) <= 0.0625 * scale
        mr, cs = pu.maxrel(dw, ref["dw"]), pu.cosine(dw, ref["dw"])
        assert mr <= pu.GRAD_MAXREL and cs > pu.GRAD_COS, ("dw", mr, cs)


@pytest.mark.parametrize("keep", [True, False])
def test_a_column_that_ties_with_the_target(keep):
    """Two identical columns of W, one of them a row's target and both that row's largest logits by far: the kernels know
    the target among a lane's values by its value, and the twin has the same value -- it must keep its say in the
    block's exponent (without it the twin's dlogit overflows the block's range)."""
    N, d, V = 512, 128, 1024
    g = torch.Generator().manual_seed(5)
    x = torch.randn(N, d, generator=g)
    w = torch.randn(d, V, generator=g) * d ** -0.5
    y = torch.randint(0, V, (N,), generator=g)
    for i0, c1, c2 in ((3, 8, 16), (200, 300, 308), (411, 900, 1016)):      # same block of 128 columns, same half of the lanes
        w[:, c1] = w[:, c2] = 10.0 * x[i0] / x[i0].pow(2).sum()
        y[i0] = c1
    inp = configs.HeadInputs("twins", x, w, y, float(x.abs().max()) / 448.0, float(w.abs().max()) / 448.0, 15.0)
    go = torch.full((N,), 1.0 / N, device="cuda")
    ours = pu.run_ours(inp, "none", x_dtype=torch.float32, w_dtype=torch.float32, grad_output=go, keep_dlogits=keep)
    assert bool(torch.isfinite(ours["dx"]).all()) and bool(torch.isfinite(ours["dw"]).all())
    ref = pu.run_oracle(inp, ours, "none", grad_output=go)
    pu.check_parity(ours, ref, "none")


@pytest.mark.parametrize("keep", [True, False])
def test_saturated_logits_under_the_largest_cap(keep):
    """cap = 40 and logits that saturate it: every row's target at +cap, everything else at -cap, so that e^{z - cap} spans
    e^{-80}.  The target, kept out of its block's exponent, still goes into the row sum at the block's scale: the sum
    must stay finite."""
    from slowrun_amd import cuda_kernels as ck
    from oracle import eager
    N, d, V = 300, 64, 700
    g = torch.Generator().manual_seed(2)
    y = torch.randint(0, V, (N,), generator=g)
    x = torch.zeros(N, d); x[:, 0] = 1.0
    w = torch.full((d, V), 0.0); w[0, :] = -400.0
    x, w, y = x.cuda(), w.cuda(), y.cuda()
    x = x + 0.0
    # row i gets +400 at its own target through hidden unit 1 + (i % 32): rows of one block of 32 have different units
    for i in range(N):
        x[i, 1 + (i % 32)] = 1.0
    w[1:33, :] = 0.0
    for i in range(N):
        w[1 + (i % 32), y[i]] = 800.0
    x_s, w_s, cap = 1.0 / 448.0 * 2.0, 800.0 / 448.0, 40.0
    go = torch.full((N,), 1.0 / N, device="cuda")
    out, saved, lse, am, nv = ck.ce_forward(x, w, y, x_s, w_s, cap, "none", keep_dlogits=keep)
    dx, dw = ck.ce_backward(saved, y, go, N, d, V, x_s, w_s, cap, 1.0, "none", torch.float32, torch.float32, keep_dlogits=keep)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(lse).all())
    assert bool(torch.isfinite(dx).all()) and bool(torch.isfinite(dw).all())
    ref = eager.softcapped_ce(x, w, y, x_s, w_s, cap=cap, reduction="none", grad_output=go)
    assert float((lse - ref["lse"]).abs().max()) <= 1e-3 * float(ref["lse"].abs().max())
