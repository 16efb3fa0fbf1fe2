"""OCP fp8 code tables in numpy (float64), written from the format definition.

e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa; no infinities; S.1111.111 is
NaN; largest finite 448; smallest subnormal 2**-9.
e5m2:   1 sign, 5 exponent (bias 15), 2 mantissa; IEEE-like inf/NaN; largest
finite 57344.

The reference quantises with ``x.div(x_s).to(torch.float8_e4m3fn)``
(tiny/cuda_kernels.py:340-341), which is round-to-nearest-even and NOT
saturating: anything that rounds past 448 becomes NaN.  encode_e4m3 restates
that rule so the HIP quantiser can be checked byte for byte.
"""
import numpy as np


def decode_e4m3_table():
    """Values of all 256 e4m3fn codes (NaN for 0x7f / 0xff)."""
    out = np.empty(256, dtype=np.float64)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 0x7
        if e == 0xF and m == 0x7:
            v = np.nan
        elif e == 0:
            v = m * 2.0 ** -9
        else:
            v = (1.0 + m / 8.0) * 2.0 ** (e - 7)
        out[c] = s * v
    return out


def decode_e5m2_table():
    out = np.empty(256, dtype=np.float64)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 2) & 0x1F
        m = c & 0x3
        if e == 0x1F:
            v = np.inf if m == 0 else np.nan
        elif e == 0:
            v = m * 2.0 ** -16
        else:
            v = (1.0 + m / 4.0) * 2.0 ** (e - 15)
        out[c] = s * v
    return out


_E4M3 = decode_e4m3_table()
_E4M3_POS = _E4M3[:0x7F]          # codes 0x00..0x7e, ascending, finite


def decode_e4m3(codes):
    return _E4M3[np.asarray(codes, dtype=np.uint8)]


def encode_e4m3(x):
    """float -> e4m3fn code, round-to-nearest-even, non-saturating.

    Magnitudes that round above 448 (> 464, the midpoint to the would-be 480)
    give NaN (0x7f | sign), as torch's cast does; so do inf and NaN.
    """
    x = np.asarray(x, dtype=np.float64)
    sign = np.where(np.signbit(x), 0x80, 0).astype(np.uint8)
    a = np.abs(x)
    hi = np.searchsorted(_E4M3_POS, a, side="left")      # first code with value >= a
    hi = np.clip(hi, 0, 0x7E)
    lo = np.clip(hi - 1, 0, 0x7E)
    dlo = np.abs(a - _E4M3_POS[lo])
    dhi = np.abs(_E4M3_POS[hi] - a)
    pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    # overflow: above 448 (mantissa 0b110) the next grid point would be 480
    # (mantissa 0b111, the NaN code).  The midpoint 464 ties to the even mantissa,
    # i.e. down to 448; anything strictly above it rounds to the NaN code.
    over = (a > 464.0) | ~np.isfinite(x)
    code = np.where(over, 0x7F, code).astype(np.uint8)
    return (code | sign).astype(np.uint8)
