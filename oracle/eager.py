"""The reference's eager loss head, restated with stock torch ops.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

What is followed, line by line (paths relative to the reference checkout):
  tiny/cuda_kernels.py:340-341   x_f8 = x.div(x_s).to(float8_e4m3fn); same for W
  tiny/train.py:496-497          logits = x @ W with W stored (d, V)
  tiny/train.py:742              logits = cap * tanh(logits / cap)
  tiny/train.py:743              F.cross_entropy(logits, targets, ignore_index=-1,
                                                 reduction=...)
  tiny/cuda_kernels.py:226-240   MTP: loss_i = sum_k w_k (lse_i - z[i, y[i+k]])
  tiny/cuda_kernels.py:414       grads are returned for the *unquantised* x and W
                                 (straight-through), nothing else gets a grad.

Two deliberate differences from tiny/train.py:741: every column of W takes part
(no slice to 50257), and the matmul runs in fp32 on the dequantised fp8 values
rather than in autocast bf16.

Everything is row-chunked: the N x V logits of one chunk exist at a time, so the
full benchmark shapes can be evaluated on a GPU with torch or on the CPU.
"""
import math

import torch
import torch.nn.functional as F

IGNORE_INDEX = -1


def quantize_e4m3(t, scale):
    """tiny/cuda_kernels.py:340-341 - per-tensor scaled, RNE, non-saturating.

    The library's own division: for a Python-float scale torch's GPU kernels compute t * (1 / scale) with the
    reciprocal taken once in fp32, its CPU kernels divide element by element.  The two differ in the last bit for
    about one value in 10^5, which matters only where the quotient lands on an fp8 rounding tie; the reference
    runs this line on the GPU."""
    return t.div(scale).to(torch.float8_e4m3fn)


def dequantize(q, scale):
    return q.to(torch.float32) * scale


def _softcap(u, cap):
    return cap * torch.tanh(u / cap)          # tiny/train.py:742


def softcapped_ce(x, w, targets, x_s=None, w_s=None, cap=15.0, reduction="mean",
                  grad_output=None, want_grads=True, row_chunk=2048, dtype=torch.float32):
    """Eager softcapped cross-entropy forward (+ autograd backward).

    x (N, d), w (d, V), targets (N,) int64 with IGNORE_INDEX = -1.
    x_s / w_s: fp8 scales (python floats); None disables quantisation (the
    plain fp32 plumbing case).
    reduction 'mean' -> scalar (sum over valid rows / n_valid, NaN if none valid,
    as F.cross_entropy gives); 'none' -> (N,) with 0 at ignored rows.
    grad_output: upstream gradient; scalar for 'mean' (default 1), (N,) for
    'none' (default 1/N each, i.e. the caller's ``.mean()``, tiny/train.py:1417).

    Returns dict(loss, lse, argmax, dx, dw, n_valid).  dx, dw are fp32 (`dtype`).
    """
    N, d = x.shape
    V = w.shape[1]
    dev = x.device
    if x_s is not None:
        xq = dequantize(quantize_e4m3(x, x_s), x_s).to(dtype)
        wq = dequantize(quantize_e4m3(w, w_s), w_s).to(dtype)
    else:
        xq, wq = x.to(dtype), w.to(dtype)
    n_valid = int((targets != IGNORE_INDEX).sum())
    if grad_output is None:
        grad_output = 1.0 if reduction == "mean" else torch.full((N,), 1.0 / N, dtype=dtype, device=dev)
    wleaf = wq.detach().clone().requires_grad_(want_grads)
    losses = torch.empty(N, dtype=dtype, device=dev)
    lse = torch.empty(N, dtype=dtype, device=dev)
    argmax = torch.empty(N, dtype=torch.int64, device=dev)
    dx = torch.zeros(N, d, dtype=dtype, device=dev) if want_grads else None
    for r0 in range(0, N, row_chunk):
        r1 = min(N, r0 + row_chunk)
        xc = xq[r0:r1].detach().clone().requires_grad_(want_grads)
        with torch.set_grad_enabled(want_grads):
            u = xc @ wleaf                                   # tiny/train.py:497
            z = _softcap(u, cap)
            li = F.cross_entropy(z, targets[r0:r1], ignore_index=IGNORE_INDEX, reduction="none")
        losses[r0:r1] = li.detach()
        lse[r0:r1] = torch.logsumexp(z.detach(), dim=1)
        argmax[r0:r1] = u.detach().argmax(dim=1)
        if want_grads:
            if reduction == "mean":
                if n_valid > 0:
                    (li.sum() * (float(grad_output) / n_valid)).backward()
            else:
                (li * grad_output[r0:r1]).sum().backward()
            if xc.grad is not None:
                dx[r0:r1] = xc.grad
    if reduction == "mean":
        loss = losses.sum() / n_valid if n_valid > 0 else torch.tensor(float("nan"), dtype=dtype, device=dev)
    else:
        loss = losses
    dw = None
    if want_grads:
        dw = wleaf.grad if wleaf.grad is not None else torch.zeros_like(wleaf)
    return dict(loss=loss, losses=losses, lse=lse, argmax=argmax, dx=dx, dw=dw, n_valid=n_valid)


def rms_norm(h, eps=None):
    """F.rms_norm(h, (d,)) without weight (tiny/train.py:397-398) in fp32 with one rounding to h's dtype, which
    is what torch computes for bf16 input; eps=None is torch's default, the machine epsilon of the type it
    computes in (float32 for bf16 and fp32 input).  Returns (normalised rows in h's dtype, rstd (N, 1) in fp32)."""
    eps = torch.finfo(torch.float64 if h.dtype == torch.float64 else torch.float32).eps if eps is None else eps
    hf = h.float()
    rstd = torch.rsqrt(hf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return (hf * rstd).to(h.dtype), rstd


def rms_norm_backward(h, rstd, g):
    """Gradient of rms_norm with respect to h for an upstream gradient g of the normalised rows:
    dh = rstd * (g - xhat * mean(g * xhat)), xhat = h * rstd."""
    xhat = h.float() * rstd
    gf = g.float()
    return rstd * (gf - xhat * (gf * xhat).mean(dim=-1, keepdim=True))


def norm_softcapped_ce(h, w, targets, x_s, w_s, cap=15.0, reduction="mean", eps=None, **kw):
    """The trunk's final norm followed by the head (tiny/train.py:734 then :682-696): softcapped_ce on
    rms_norm(h), with the head's gradient (rounded to h's dtype, as the unfused path stores it) taken back
    through the norm.  Returns softcapped_ce's dict with dx replaced by the gradient with respect to h."""
    x, rstd = rms_norm(h, eps)
    res = softcapped_ce(x, w, targets, x_s, w_s, cap, reduction, **kw)
    if res["dx"] is not None:
        res["dx_normalised"] = res["dx"]
        res["dx"] = rms_norm_backward(h, rstd, res["dx"].to(h.dtype))
    res["x"] = x
    return res


def softcapped_ce_mtp(x, w, targets, mtp_weights, x_s=None, w_s=None, cap=15.0,
                      grad_output=None, want_grads=True, row_chunk=2048, dtype=torch.float32):
    """Multi-token-prediction variant, reduction 'none' (tiny/cuda_kernels.py:226-240).

    loss_i = sum_k w_k * CE(z_i, y[i+k]); offset k takes part when i+k < N and
    y[i+k] != -1.  Offsets index the flattened target vector, as the reference
    kernel does (tiny/cuda_kernels.py:229).
    """
    N, d = x.shape
    dev = x.device
    if x_s is not None:
        xq = dequantize(quantize_e4m3(x, x_s), x_s).to(dtype)
        wq = dequantize(quantize_e4m3(w, w_s), w_s).to(dtype)
    else:
        xq, wq = x.to(dtype), w.to(dtype)
    mtp_weights = torch.as_tensor(mtp_weights, dtype=dtype, device=dev)
    K = mtp_weights.numel()
    if grad_output is None:
        grad_output = torch.full((N,), 1.0 / N, dtype=dtype, device=dev)
    shifted = []
    for k in range(K):
        t = torch.full((N,), IGNORE_INDEX, dtype=torch.int64, device=dev)
        if k < N:                      # (fewer rows than offsets: the later offsets have no row to point at)
            t[: N - k] = targets[k:]
        shifted.append(t)
    wleaf = wq.detach().clone().requires_grad_(want_grads)
    losses = torch.empty(N, dtype=dtype, device=dev)
    dx = torch.zeros(N, d, dtype=dtype, device=dev) if want_grads else None
    for r0 in range(0, N, row_chunk):
        r1 = min(N, r0 + row_chunk)
        xc = xq[r0:r1].detach().clone().requires_grad_(want_grads)
        with torch.set_grad_enabled(want_grads):
            z = _softcap(xc @ wleaf, cap)
            li = 0
            for k in range(K):
                li = li + mtp_weights[k] * F.cross_entropy(z, shifted[k][r0:r1], ignore_index=IGNORE_INDEX,
                                                           reduction="none")
        losses[r0:r1] = li.detach()
        if want_grads:
            (li * grad_output[r0:r1]).sum().backward()
            if xc.grad is not None:
                dx[r0:r1] = xc.grad
    dw = (wleaf.grad if wleaf.grad is not None else torch.zeros_like(wleaf)) if want_grads else None
    return dict(loss=losses, losses=losses, dx=dx, dw=dw)


def ln(v):
    return math.log(v)
