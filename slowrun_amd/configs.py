"""Synthetic inputs for the five benchmark shapes of the loss-head path.

Everything is drawn on the CPU in fp32 from ``torch.Generator().manual_seed(seed)``
in a fixed order (X, then W, then targets, then masks) and only then cast or
moved, so a CPU checker and the GPU path see identical bits.  W has the
``(d, V)`` layout of the reference's ``CastedLinearT`` (tiny/train.py:489-497);
targets are int64 with ``-1`` meaning "ignore" (tiny/train.py:743); the default
cap values are the reference's (tiny/train.py:742).

name            N      d     V       cap  notes
cpu_plumbing    2048   768   50304   15   fp32, no fp8 (scales None)
tiny_track      32768  1024  50304   15   amax fp8 scales
limited_2p7b    65536  2560  50304   15   X x1.5, W ~ N(0,1/d), Zipf(1.1) targets
large_vocab     16384  4096  131072  30   targets uniform over all V
irregular       30011  2560  50304   15   12% ignored, 0.1% rows x50
"""
from dataclasses import dataclass

import torch
import torch.nn.functional as F

REAL_VOCAB = 50257          # GPT-2 vocabulary; 50304 is its padding to a multiple of 64 (tiny/train.py:505)


@dataclass
class HeadInputs:
    name: str
    x: torch.Tensor            # (N, d) fp32
    w: torch.Tensor            # (d, V) fp32
    targets: torch.Tensor      # (N,) int64
    x_s: float | None
    w_s: float | None
    cap: float

    @property
    def shape(self):
        return self.x.shape[0], self.x.shape[1], self.w.shape[1]


SHAPES = {
    "cpu_plumbing": dict(seed=0, N=2048, d=768, V=50304, cap=15.0),
    "tiny_track": dict(seed=1, N=32768, d=1024, V=50304, cap=15.0),
    "limited_2p7b": dict(seed=2, N=65536, d=2560, V=50304, cap=15.0),
    "large_vocab": dict(seed=3, N=16384, d=4096, V=131072, cap=30.0),
    "irregular": dict(seed=4, N=30011, d=2560, V=50304, cap=15.0),
}


def _amax_scale(t):
    return float(t.abs().max()) / 448.0


def make_inputs(name, N=None, d=None, V=None):
    """Build one configuration; N/d/V may be overridden to get a reduced case
    with the same distributions and draw order."""
    cfg = dict(SHAPES[name])
    N = cfg["N"] if N is None else N
    d = cfg["d"] if d is None else d
    V = cfg["V"] if V is None else V
    g = torch.Generator().manual_seed(cfg["seed"])
    x = F.rms_norm(torch.randn(N, d, generator=g), (d,))
    hi = min(REAL_VOCAB, V)
    if name == "cpu_plumbing":
        w = 0.02 * torch.randn(d, V, generator=g)
        y = torch.randint(0, hi, (N,), generator=g)
        return HeadInputs(name, x, w, y, None, None, cfg["cap"])
    if name == "tiny_track":
        w = 0.02 * torch.randn(d, V, generator=g)
        y = torch.randint(0, hi, (N,), generator=g)
    elif name == "limited_2p7b":
        x = 1.5 * x
        w = torch.randn(d, V, generator=g) * d ** -0.5
        p = (torch.arange(hi, dtype=torch.float64) + 1.0) ** -1.1
        y = torch.multinomial(p / p.sum(), N, True, generator=g)
    elif name == "large_vocab":
        w = torch.randn(d, V, generator=g) * d ** -0.5
        y = torch.randint(0, V, (N,), generator=g)
    elif name == "irregular":
        w = torch.randn(d, V, generator=g) * d ** -0.5
        y = torch.randint(0, hi, (N,), generator=g)
        hot = torch.rand(N, generator=g) < 0.001
        x[hot] *= 50.0
        y[torch.rand(N, generator=g) < 0.12] = -1
    else:
        raise KeyError(name)
    return HeadInputs(name, x, w, y, _amax_scale(x), _amax_scale(w), cfg["cap"])
