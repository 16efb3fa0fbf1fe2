"""Drop-in for the reference's ``tiny/cuda_kernels.py`` on MI355X.

Exports the same names the trainer imports (tiny/train.py:47):

    from cuda_kernels import CE_KERNEL_VOCAB_SIZE, FusedSoftcappedCrossEntropy

``FusedSoftcappedCrossEntropy.apply(x, targets, mtp_weights, lm_head_weight, x_s,
w_s, grad_s, grad_scale[, cap])`` keeps the positional signature of
tiny/cuda_kernels.py:338 and returns the per-row losses (N,), which the caller
reduces with ``.mean()`` (tiny/train.py:1417).  Underneath, the work is done by the
HIP kernels of libslowrun_ce.so through its C ABI; the N x V logits are never
stored.  What is kept for backward depends on KEEP_DLOGITS (below): by default the
forward pass leaves the dlogits in the saved state, 8 bits per logit (N x V bytes,
3.3 GB at N = 65536, V = 50304; the reference keeps three times that,
tiny/cuda_kernels.py:359-371), and backward is two GEMMs; with keep_dlogits=False
nothing N x V sized is kept and backward computes the logit tiles again.

Differences from the reference that a caller can see:
  * V is a runtime size (CE_KERNEL_VOCAB_SIZE is kept only for the trainer's asserts);
  * ``reduction='mean'`` is available (mean over rows whose target is not -1, like
    F.cross_entropy(ignore_index=-1) in the eager head, tiny/train.py:743);
  * rows with target -1 give loss 0 and zero gradient;
  * up to 4 multi-token-prediction offsets (``mtp_weights``), with the offsets that run past
    the end of the target vector or hit a -1 target left out of both the loss and the gradient
    (the reference kernel leaves them out of the loss only, tiny/cuda_kernels.py:233,242-246);
  * ``grad_s`` is accepted and unused: the reference needs it to fit dlogits into
    e5m2 (tiny/cuda_kernels.py:265); here each row of the on-chip dlogits carries its
    own scale;
  * dW is returned in the weight's dtype and uses the upstream gradient of every row,
    not its mean (tiny/cuda_kernels.py:412 assumes it is uniform).
"""
import ctypes as C
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import SceArgs, SceShape

CE_KERNEL_VOCAB_SIZE = 50304          # tiny/cuda_kernels.py:82
IGNORE_INDEX = -1                     # tiny/train.py:743

# How backward gets the dlogits when a call does not say (keep_dlogits=None):
#   True   forward leaves them in the saved state, 8 bits per logit (N x V bytes held until backward; the reference
#          holds 3 N x V bytes, tiny/cuda_kernels.py:359-371); backward is two GEMMs
#   False  backward computes the logit tiles again: nothing N x V is held, backward is three GEMMs
KEEP_DLOGITS = True

_DTYPES = {torch.float32: _lib.SCE_F32, torch.bfloat16: _lib.SCE_BF16}


def _scale_value(s, like):
    """A scale as the C ABI takes it: a Python float, or -- for a one-element tensor on ``like``'s device -- that tensor
    as float32, which the kernels read when they run (no host read, so the value may come from earlier work on the
    stream, e.g. ``amax_scale``, and may change between replays of a captured graph).  A tensor on the CPU is read here."""
    if isinstance(s, torch.Tensor):
        if s.numel() != 1:
            raise ValueError("a scale must have one element")
        if s.device.type != "cuda":
            return float(s)
        return s.detach().to(dtype=torch.float32).reshape(())
    return float(s)


def _split_scale(s):
    """(float, None) for a host scale, (1.0, tensor) for a device scale: the two slots of the custom ops' signatures."""
    return (1.0, s) if isinstance(s, torch.Tensor) else (s, None)


def _set_scales(a, x_s, w_s):
    """Fills x_s / w_s or x_s_dev / w_s_dev of an SceArgs; returns the tensors that must stay alive over the call."""
    keep = []
    for name, s in (("x_s", x_s), ("w_s", w_s)):
        if isinstance(s, torch.Tensor):
            setattr(a, name, 1.0)
            setattr(a, name + "_dev", s.data_ptr())
            keep.append(s)
        else:
            setattr(a, name, s)
    return keep


def _dtype_code(t, what):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"{what} must be float32 or bfloat16, got {t.dtype}") from None


def _stream_ptr(device):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _mtp(mtp_weights, device):
    """(n_predict, float32 device tensor or None).  None means a single offset of weight 1."""
    if mtp_weights is None:
        return 1, None
    w = mtp_weights.detach().to(device=device, dtype=torch.float32).contiguous().reshape(-1)
    if not 1 <= w.numel() <= 4:
        raise ValueError(f"mtp_weights must hold 1 to 4 offsets, got {w.numel()}")
    return w.numel(), w


def _base_args(x_like, N, d, V, x_s, w_s, cap, grad_scale, reduction, targets, n_predict=1, mtp_w=None):
    a = SceArgs()
    a.struct_size = C.sizeof(SceArgs)
    a.device = x_like.device.index if x_like.device.index is not None else torch.cuda.current_device()
    a.stream = _stream_ptr(x_like.device)
    a.shape = SceShape(N, d, V, n_predict, 0)
    a.targets = targets.data_ptr()
    a.mtp_weights = mtp_w.data_ptr() if mtp_w is not None else None
    a._scale_refs = _set_scales(a, x_s, w_s)
    a.cap, a.grad_scale = cap, grad_scale
    a.ignore_index = IGNORE_INDEX
    a.reduction = _lib.SCE_REDUCE_MEAN if reduction == "mean" else _lib.SCE_REDUCE_NONE
    return a


def _check_inputs(x, w, targets):
    if not x.is_cuda:
        raise RuntimeError("FusedSoftcappedCrossEntropy runs on an MI355X GPU only; got a CPU tensor")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[0]:
        raise ValueError(f"expected x (N, d) and lm_head_weight (d, V), got {tuple(x.shape)} and {tuple(w.shape)}")
    if targets.dim() != 1 or targets.shape[0] != x.shape[0] or targets.dtype != torch.int64:
        raise ValueError("targets must be int64 of shape (N,)")


class WeightCache:
    """The two e4m3 copies of the LM-head weight, kept across calls.

    The reference re-quantises and re-lays-out W on every micro-step (tiny/cuda_kernels.py:341-343) although W
    only changes at optimizer.step().  With a WeightCache the forward quantises W only when the tensor (storage,
    version counter, shape, dtype, scale) differs from the one the cache was filled from.

    The version counter does not see everything: writes through ``w.data`` (the reference broadcasts parameters
    that way, tiny/train.py:1586), a checkpoint loaded with ``copy_`` into ``.data``, or a new tensor that happens
    to be allocated at the old address.  Call ``invalidate()`` after anything of that kind -- after
    ``optimizer.step()`` is always right.  ``generation`` counts the fills; ce_forward hands it out with the saved
    state and ce_backward refuses a cache that has been refilled since, instead of using another W's bytes.
    """

    def __init__(self):
        self.buf = None
        self.key = None
        self.generation = 0

    def invalidate(self):
        """The next forward quantises W again, whatever the tensor's version counter says."""
        self.key = None

    def prepare(self, w, w_s, nbytes):
        """Returns (buffer, valid)."""
        skey = (w_s.data_ptr(), w_s._version) if isinstance(w_s, torch.Tensor) else float(w_s)
        key = (w.data_ptr(), w._version, tuple(w.shape), w.dtype, skey, w.device)
        if self.buf is None or self.buf.numel() < nbytes or self.buf.device != w.device:
            self.buf = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
            self.key = None
        valid = self.key == key
        if not valid:
            self.generation += 1
        self.key = key
        return self.buf, valid


def ce_forward(x, w, targets, x_s, w_s, cap, reduction, want_argmax=False, mtp_weights=None, vocab_size=None,
               weight_cache=None, norm_eps=None, keep_dlogits=False, no_alloc=False, operand_dtype=None):
    """One call of sce_forward.  Returns (out, saved, lse, argmax, n_valid).

    operand_dtype: None / torch.float8_e4m3fn (the fused path's e4m3 operands) or torch.bfloat16 (the arithmetic of the
    eager head under bf16 autocast: bf16 operands, logits rounded to bf16; forward only, the scales are not used).
    no_alloc: call sce_forward_noalloc instead, which keeps its scratch in a static device array of the library (this
    wrapper still allocates the outputs with torch; a caller that may not allocate passes buffers of its own to the C ABI).

    keep_dlogits: the forward pass also leaves the dlogits in ``saved`` (pass the same value to ce_backward).

    norm_eps: when given, ``x`` is the hidden state before the trunk's final ``F.rms_norm(x, (d,))``
    (tiny/train.py:397-398,734) and the norm is applied inside the quantiser."""
    _check_inputs(x, w, targets)
    n_predict, mtp_w = _mtp(mtp_weights, x.device)
    if n_predict > 1 and reduction != "none":
        raise ValueError("multi-token prediction returns per-row losses: use reduction='none'")
    x = x if x.stride(1) == 1 else x.contiguous()
    w = w if w.stride(1) == 1 else w.contiguous()
    targets = targets.contiguous()
    N, d = x.shape
    V = w.shape[1]
    dev = x.device
    sz = _lib.sizes_for(N, d, V, n_predict)
    bf16_ops = operand_dtype == torch.bfloat16
    if operand_dtype not in (None, torch.float8_e4m3fn, torch.bfloat16):
        raise TypeError(f"operand_dtype must be float8_e4m3fn or bfloat16, got {operand_dtype}")
    if bf16_ops:
        if keep_dlogits or weight_cache is not None or norm_eps is not None:
            raise ValueError("bf16 operands are for the forward-only eval head: no kept dlogits, weight cache or fused norm")
        x_s = w_s = 1.0
    saved = torch.empty(sz.saved_bf16_bytes if bf16_ops else
                        (sz.saved_x_bytes if weight_cache is not None else sz.saved_bytes) + (sz.dlogits_bytes if keep_dlogits else 0),
                        dtype=torch.uint8, device=dev)
    ws = None if no_alloc else torch.empty(sz.fwd_workspace_bytes, dtype=torch.uint8, device=dev)
    losses = torch.empty(N, dtype=torch.float32, device=dev)
    lse = torch.empty(N, dtype=torch.float32, device=dev)
    loss = torch.empty(1, dtype=torch.float32, device=dev)
    n_valid = torch.empty(2, dtype=torch.int32, device=dev)
    argmax = torch.empty(N, dtype=torch.int32, device=dev) if want_argmax else None
    a = _base_args(x, N, d, V, x_s, w_s, cap, 1.0, reduction, targets, n_predict, mtp_w)
    a.x, a.x_dtype, a.x_ld = x.data_ptr(), _dtype_code(x, "x"), x.stride(0)
    a.w, a.w_dtype, a.w_ld = w.data_ptr(), _dtype_code(w, "lm_head_weight"), w.stride(0)
    a.loss, a.losses, a.lse, a.n_valid = loss.data_ptr(), losses.data_ptr(), lse.data_ptr(), n_valid.data_ptr()
    a.argmax = argmax.data_ptr() if want_argmax else None
    a.saved, a.saved_bytes = saved.data_ptr(), saved.numel()
    if ws is not None:
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    a.vocab_limit = 0 if vocab_size is None else int(vocab_size)
    a.dlogits_from_forward = int(bool(keep_dlogits))
    a.operand_dtype = _lib.SCE_BF16 if bf16_ops else 0
    if norm_eps is not None:
        a.norm, a.norm_eps = 1, float(norm_eps)
    if weight_cache is not None:
        wbuf, valid = weight_cache.prepare(w, w_s, sz.wcache_bytes)
        a.wcache, a.wcache_bytes, a.wcache_valid = wbuf.data_ptr(), wbuf.numel(), int(valid)
    if no_alloc:
        _lib.check(_lib.lib().sce_forward_noalloc(C.byref(a)), "sce_forward_noalloc")
    else:
        _lib.check(_lib.lib().sce_forward(C.byref(a)), "sce_forward")
    out = loss.reshape(()) if reduction == "mean" else losses
    return out, saved, lse, argmax, n_valid


def ce_backward(saved, targets, grad_output, N, d, V, x_s, w_s, cap, grad_scale, reduction, x_dtype, w_dtype,
                panel_rows=0, workspace_bytes=None, mtp_weights=None, vocab_size=None, weight_cache=None,
                hidden=None, norm_eps=None, keep_dlogits=False, cache_generation=None):
    """One call of sce_backward.  Returns (dx (N,d) in x_dtype, dw (d,V) in w_dtype).

    hidden, norm_eps: the pre-norm hidden state and eps given to ce_forward(norm_eps=...); dx is then the
    gradient with respect to that hidden state.
    cache_generation: ``weight_cache.generation`` as it was right after the matching ce_forward; checked."""
    dev = saved.device
    n_predict, mtp_w = _mtp(mtp_weights, dev)
    sz = _lib.sizes_for(N, d, V, n_predict)
    nbytes = (sz.bwd_workspace_kept_bytes if keep_dlogits else sz.bwd_workspace_bytes) if workspace_bytes is None else workspace_bytes
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    dx = torch.empty(N, d, dtype=x_dtype, device=dev)
    dw = torch.empty(d, V, dtype=w_dtype, device=dev)
    go = grad_output.detach().to(torch.float32).contiguous().reshape(-1)
    if reduction == "mean":
        if go.numel() != 1:
            raise ValueError("grad_output must be a scalar for reduction='mean'")
    elif go.numel() != N:
        raise ValueError("grad_output must have one element per row for reduction='none'")
    a = _base_args(saved, N, d, V, x_s, w_s, cap, grad_scale, reduction, targets, n_predict, mtp_w)
    a.saved, a.saved_bytes = saved.data_ptr(), saved.numel()
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    a.grad_output = go.data_ptr()
    a.dx, a.dx_dtype, a.dx_ld = dx.data_ptr(), _DTYPES[x_dtype], d
    a.dw, a.dw_dtype, a.dw_ld = dw.data_ptr(), _DTYPES[w_dtype], V
    a.panel_rows = panel_rows
    a.vocab_limit = 0 if vocab_size is None else int(vocab_size)
    a.dlogits_from_forward = int(bool(keep_dlogits))
    if norm_eps is not None:
        if hidden is None or tuple(hidden.shape) != (N, d) or hidden.device != dev:
            raise ValueError("backward through the fused norm needs the (N, d) hidden state given to forward")
        hidden = hidden if hidden.stride(1) == 1 else hidden.contiguous()
        a.norm, a.norm_eps = 1, float(norm_eps)
        a.x, a.x_dtype, a.x_ld = hidden.data_ptr(), _dtype_code(hidden, "hidden"), hidden.stride(0)
    if weight_cache is not None:
        if cache_generation is not None and cache_generation != weight_cache.generation:
            raise RuntimeError("the weight cache has been refilled since the forward pass this backward belongs to "
                               f"(generation {weight_cache.generation}, forward saw {cache_generation})")
        a.wcache, a.wcache_bytes, a.wcache_valid = weight_cache.buf.data_ptr(), weight_cache.buf.numel(), 1
    _lib.check(_lib.lib().sce_backward(C.byref(a)), "sce_backward")
    return dx, dw


# ---------------------------------------------------------------------------------------------
# torch.library custom ops, so that a torch.compile'd model (tiny/train.py:1254) traces the loss head
# as two opaque calls instead of breaking the graph; the reference wraps its kernel the same way
# (tiny/cuda_kernels.py:314).  The fake implementations only describe shapes and dtypes.
# ---------------------------------------------------------------------------------------------
@torch.library.custom_op("slowrun_amd::ce_forward", mutates_args=())
def ce_forward_op(x: torch.Tensor, w: torch.Tensor, targets: torch.Tensor, mtp_weights: Optional[torch.Tensor],
                  x_s: float, w_s: float, cap: float, mean: bool, keep: bool,
                  x_s_t: Optional[torch.Tensor] = None, w_s_t: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    out, saved, _lse, _am, _nv = ce_forward(x, w, targets, x_s if x_s_t is None else x_s_t, w_s if w_s_t is None else w_s_t, cap,
                                            "mean" if mean else "none", mtp_weights=mtp_weights, keep_dlogits=keep)
    return out, saved


@ce_forward_op.register_fake
def _ce_forward_fake(x, w, targets, mtp_weights, x_s, w_s, cap, mean, keep, x_s_t=None, w_s_t=None):
    N, d = x.shape
    V = w.shape[1]
    n_predict = 1 if mtp_weights is None else mtp_weights.numel()
    sz = _lib.sizes_for(N, d, V, n_predict)
    out = x.new_empty((), dtype=torch.float32) if mean else x.new_empty((N,), dtype=torch.float32)
    return out, x.new_empty((sz.saved_bytes + (sz.dlogits_bytes if keep else 0),), dtype=torch.uint8)


@torch.library.custom_op("slowrun_amd::ce_backward", mutates_args=())
def ce_backward_op(saved: torch.Tensor, targets: torch.Tensor, grad_output: torch.Tensor, mtp_weights: Optional[torch.Tensor],
                   N: int, d: int, V: int, x_s: float, w_s: float, cap: float, grad_scale: float, mean: bool,
                   x_bf16: bool, w_bf16: bool, keep: bool,
                   x_s_t: Optional[torch.Tensor] = None, w_s_t: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    return ce_backward(saved, targets, grad_output, N, d, V, x_s if x_s_t is None else x_s_t, w_s if w_s_t is None else w_s_t, cap,
                       grad_scale, "mean" if mean else "none",
                       torch.bfloat16 if x_bf16 else torch.float32, torch.bfloat16 if w_bf16 else torch.float32,
                       mtp_weights=mtp_weights, keep_dlogits=keep)


@ce_backward_op.register_fake
def _ce_backward_fake(saved, targets, grad_output, mtp_weights, N, d, V, x_s, w_s, cap, grad_scale, mean, x_bf16, w_bf16, keep,
                      x_s_t=None, w_s_t=None):
    return (saved.new_empty((N, d), dtype=torch.bfloat16 if x_bf16 else torch.float32),
            saved.new_empty((d, V), dtype=torch.bfloat16 if w_bf16 else torch.float32))


@torch.library.custom_op("slowrun_amd::norm_ce_forward", mutates_args=())
def norm_ce_forward_op(h: torch.Tensor, w: torch.Tensor, targets: torch.Tensor, mtp_weights: Optional[torch.Tensor],
                       x_s: float, w_s: float, cap: float, mean: bool, eps: float, keep: bool,
                       x_s_t: Optional[torch.Tensor] = None, w_s_t: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    out, saved, _lse, _am, _nv = ce_forward(h, w, targets, x_s if x_s_t is None else x_s_t, w_s if w_s_t is None else w_s_t, cap,
                                            "mean" if mean else "none", mtp_weights=mtp_weights, norm_eps=eps, keep_dlogits=keep)
    return out, saved


norm_ce_forward_op.register_fake(lambda h, w, targets, mtp_weights, x_s, w_s, cap, mean, eps, keep, x_s_t=None, w_s_t=None:
                                 _ce_forward_fake(h, w, targets, mtp_weights, x_s, w_s, cap, mean, keep))


@torch.library.custom_op("slowrun_amd::norm_ce_backward", mutates_args=())
def norm_ce_backward_op(saved: torch.Tensor, h: torch.Tensor, targets: torch.Tensor, grad_output: torch.Tensor,
                        mtp_weights: Optional[torch.Tensor], V: int, x_s: float, w_s: float, cap: float, grad_scale: float,
                        mean: bool, w_bf16: bool, eps: float, keep: bool,
                        x_s_t: Optional[torch.Tensor] = None, w_s_t: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    N, d = h.shape
    return ce_backward(saved, targets, grad_output, N, d, V, x_s if x_s_t is None else x_s_t, w_s if w_s_t is None else w_s_t, cap,
                       grad_scale, "mean" if mean else "none",
                       h.dtype, torch.bfloat16 if w_bf16 else torch.float32, mtp_weights=mtp_weights, hidden=h, norm_eps=eps,
                       keep_dlogits=keep)


@norm_ce_backward_op.register_fake
def _norm_ce_backward_fake(saved, h, targets, grad_output, mtp_weights, V, x_s, w_s, cap, grad_scale, mean, w_bf16, eps, keep,
                           x_s_t=None, w_s_t=None):
    return torch.empty_like(h), h.new_empty((h.shape[1], V), dtype=torch.bfloat16 if w_bf16 else torch.float32)


class FusedSoftcappedCrossEntropy(torch.autograd.Function):
    """Same call as tiny/cuda_kernels.py:336-414; see the module docstring."""

    @staticmethod
    def forward(ctx, x, targets, mtp_weights, lm_head_weight, x_s, w_s, grad_s, grad_scale, cap=15.0, reduction="none",
                keep_dlogits=None):
        if reduction not in ("none", "mean"):
            raise ValueError("reduction must be 'none' or 'mean'")
        _dtype_code(x, "x")
        _dtype_code(lm_head_weight, "lm_head_weight")
        xs, ws_ = _scale_value(x_s, x), _scale_value(w_s, lm_head_weight)
        (xs, xst), (ws_, wst) = _split_scale(xs), _split_scale(ws_)
        keep = bool(KEEP_DLOGITS if keep_dlogits is None else keep_dlogits)
        out, saved = ce_forward_op(x.detach(), lm_head_weight.detach(), targets, mtp_weights, xs, ws_, float(cap),
                                   reduction == "mean", keep, xst, wst)
        ctx.scale_tensors = (xst, wst)
        ctx.save_for_backward(saved, targets, mtp_weights if mtp_weights is not None else torch.empty(0, device=x.device))
        ctx.params = (x.shape[0], x.shape[1], lm_head_weight.shape[1], xs, ws_, float(cap), float(grad_scale),
                      reduction == "mean", x.dtype == torch.bfloat16, lm_head_weight.dtype == torch.bfloat16,
                      mtp_weights is not None, keep)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        saved, targets, mtp_w = ctx.saved_tensors
        N, d, V, xs, ws_, cap, gscale, mean, x_bf16, w_bf16, has_mtp, keep = ctx.params
        dx, dw = ce_backward_op(saved, targets, grad_output.contiguous(), mtp_w if has_mtp else None, N, d, V, xs, ws_, cap,
                                gscale, mean, x_bf16, w_bf16, keep, *ctx.scale_tensors)
        return dx, None, None, dw, None, None, None, None, None, None, None


class FusedNormSoftcappedCrossEntropy(torch.autograd.Function):
    """``FusedSoftcappedCrossEntropy.apply(F.rms_norm(h, (d,), eps=eps), ...)`` in one call: the trunk's final norm
    (tiny/train.py:397-398,734) runs inside the quantiser, so the normalised activations are never written, and
    backward returns the gradient with respect to ``h``.  ``eps=None`` is torch's default, float32's machine
    epsilon for bf16 and fp32 input.  Same argument order as FusedSoftcappedCrossEntropy with ``h`` in place of ``x``."""

    @staticmethod
    def forward(ctx, h, targets, mtp_weights, lm_head_weight, x_s, w_s, grad_s, grad_scale, cap=15.0, reduction="none",
                eps=None, keep_dlogits=None):
        if reduction not in ("none", "mean"):
            raise ValueError("reduction must be 'none' or 'mean'")
        _dtype_code(h, "h")
        _dtype_code(lm_head_weight, "lm_head_weight")
        eps = float(torch.finfo(torch.float32).eps if eps is None else eps)
        xs, ws_ = _scale_value(x_s, h), _scale_value(w_s, lm_head_weight)
        (xs, xst), (ws_, wst) = _split_scale(xs), _split_scale(ws_)
        hd = h.detach()
        keep = bool(KEEP_DLOGITS if keep_dlogits is None else keep_dlogits)
        out, saved = norm_ce_forward_op(hd, lm_head_weight.detach(), targets, mtp_weights, xs, ws_, float(cap),
                                        reduction == "mean", eps, keep, xst, wst)
        ctx.scale_tensors = (xst, wst)
        ctx.save_for_backward(saved, hd, targets, mtp_weights if mtp_weights is not None else torch.empty(0, device=h.device))
        ctx.params = (lm_head_weight.shape[1], xs, ws_, float(cap), float(grad_scale), reduction == "mean",
                      lm_head_weight.dtype == torch.bfloat16, mtp_weights is not None, eps, keep)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        saved, h, targets, mtp_w = ctx.saved_tensors
        V, xs, ws_, cap, gscale, mean, w_bf16, has_mtp, eps, keep = ctx.params
        dh, dw = norm_ce_backward_op(saved, h, targets, grad_output.contiguous(), mtp_w if has_mtp else None, V, xs, ws_, cap,
                                     gscale, mean, w_bf16, eps, keep, *ctx.scale_tensors)
        return dh, None, None, dw, None, None, None, None, None, None, None, None


def softcapped_cross_entropy(x, lm_head_weight, targets, x_s=None, w_s=None, cap=15.0, vocab_size=None, reduction="mean",
                             norm_eps=None, operand_dtype=None):
    """Forward-only loss of the eager head (tiny/train.py:741-743) on the fused kernel:
    ``F.cross_entropy(cap * tanh((x @ W)[..., :vocab_size] / cap), targets, ignore_index=-1, reduction=...)``; the
    N x V logits are never stored.  ``operand_dtype=torch.bfloat16`` computes what the reference's eval computes -- a bf16
    matmul (CastedLinearT under autocast, tiny/train.py:496-497) whose bf16 result goes through the softcap in fp32 -- so
    that validation losses compare; the default keeps the training path's e4m3 operands with scales ``x_s``, ``w_s``.  ``x`` may have leading batch dimensions.  With ``norm_eps``
    given, ``x`` is the hidden state before the final ``F.rms_norm(x, (d,), eps=norm_eps)`` (tiny/train.py:734),
    which is then applied inside the quantiser."""
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    if operand_dtype == torch.bfloat16:
        x_s = w_s = 1.0
    elif x_s is None or w_s is None:
        raise ValueError("e4m3 operands need their scales x_s and w_s")
    out, _saved, _lse, _am, _nv = ce_forward(x2.detach(), lm_head_weight.detach(), targets.reshape(-1),
                                             _scale_value(x_s, x2), _scale_value(w_s, lm_head_weight), float(cap),
                                             reduction, vocab_size=vocab_size, norm_eps=norm_eps, operand_dtype=operand_dtype)
    return out if reduction == "mean" else out.reshape(lead)


def target_probability(x, lm_head_weight, targets, x_s=None, w_s=None, cap=15.0, vocab_size=None, norm_eps=None,
                       operand_dtype=None):
    """p(target) of every row under the softcapped head, ``exp(logit[target] - logsumexp(logits))``: what the
    reference's ensemble evaluation extracts from the full N x V logits of each model before it averages the models
    (``_forward_pgt``, unlimited/train.py:1063-1069).  Here it is ``exp(-loss)`` of the per-row losses of
    ``softcapped_cross_entropy(..., reduction='none')``, same arguments; a row whose target is -1 has no target
    probability and gets 0."""
    losses = softcapped_cross_entropy(x, lm_head_weight, targets, x_s, w_s, cap, vocab_size, "none", norm_eps, operand_dtype)
    return torch.where(targets.reshape(losses.shape) == -1, torch.zeros_like(losses), torch.exp(-losses))


def quantize_e4m3(t, scale):
    """``t.div(scale).to(torch.float8_e4m3fn)`` (tiny/cuda_kernels.py:340-341) on the HIP quantiser."""
    if not t.is_cuda:
        raise RuntimeError("quantize_e4m3 needs a GPU tensor")
    t = t.contiguous()
    out = torch.empty(t.shape, dtype=torch.uint8, device=t.device)
    sv = _scale_value(scale, t)
    if isinstance(sv, torch.Tensor):            # a device scalar: divided by, as torch divides by a tensor
        _lib.check(_lib.lib().sce_quantize_e4m3_dev(t.data_ptr(), _dtype_code(t, "t"), out.data_ptr(), sv.data_ptr(), t.numel(),
                                                   t.device.index, _stream_ptr(t.device)), "sce_quantize_e4m3_dev")
    else:
        _lib.check(_lib.lib().sce_quantize_e4m3(t.data_ptr(), _dtype_code(t, "t"), out.data_ptr(), sv, t.numel(), t.device.index,
                                               _stream_ptr(t.device)), "sce_quantize_e4m3")
    return out.view(torch.float8_e4m3fn)


def amax_scale(t):
    """``t.abs().max() / 448`` as a 0-dim float32 tensor on ``t``'s device, without a host read: the per-tensor scale of
    the e4m3 cast, to be passed as ``x_s`` / ``w_s``."""
    if not t.is_cuda:
        raise RuntimeError("amax_scale needs a GPU tensor")
    t = t.contiguous()
    out = torch.empty((), dtype=torch.float32, device=t.device)
    _lib.check(_lib.lib().sce_amax_scale(t.data_ptr(), _dtype_code(t, "t"), t.numel(), out.data_ptr(), t.device.index,
                                        _stream_ptr(t.device)), "sce_amax_scale")
    return out


def transpose_copy(src, dst):
    """dst = src.T for one-byte element types (tiny/cuda_kernels.py:56-78)."""
    assert src.ndim == 2 and dst.ndim == 2
    M, Nn = src.shape
    assert dst.shape == (Nn, M), f"Expected dst shape ({Nn}, {M}), got {dst.shape}"
    if src.element_size() != 1 or dst.element_size() != 1:
        raise TypeError("transpose_copy handles one-byte element types (fp8)")
    if not (src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("transpose_copy needs contiguous tensors")
    _lib.check(_lib.lib().sce_transpose_bytes(src.data_ptr(), dst.data_ptr(), M, Nn, src.device.index,
                                             _stream_ptr(src.device)), "sce_transpose_bytes")
