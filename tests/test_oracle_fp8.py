"""Pins oracle/fp8.py and oracle/eager.quantize_e4m3 against the library cast
``Tensor.to(torch.float8_e4m3fn)`` that the reference calls
(tiny/cuda_kernels.py:340-341): all codes, all rounding midpoints, the overflow
edge and subnormals."""
import numpy as np
import torch

from oracle import eager, fp8


def _torch_encode(x):
    return torch.from_numpy(np.asarray(x, np.float32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def test_decode_all_codes():
    ours = fp8.decode_e4m3_table()
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(ours), np.isnan(ref))
    ok = ~np.isnan(ours)
    assert np.array_equal(ours[ok], ref[ok].astype(np.float64))
    # format facts: max finite 448, min subnormal 2^-9, exactly two NaN codes
    assert np.nanmax(ours) == 448.0 and ours[1] == 2.0 ** -9 and np.isnan(ours).sum() == 2


def test_decode_e5m2_all_codes():
    ours = fp8.decode_e5m2_table()
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e5m2).float().numpy()
    ok = np.isfinite(ours)
    assert np.array_equal(ok, np.isfinite(ref))
    assert np.array_equal(ours[ok], ref[ok].astype(np.float64))


def test_roundtrip_all_codes():
    t = fp8.decode_e4m3_table()
    codes = np.arange(256, dtype=np.uint8)
    fin = ~np.isnan(t)
    assert np.array_equal(fp8.encode_e4m3(t[fin]), codes[fin])


def test_encode_midpoints_and_edges():
    pos = fp8.decode_e4m3_table()[:0x7F]
    mids = (pos[:-1] + pos[1:]) / 2            # exactly representable in fp32
    below = np.nextafter(mids.astype(np.float32), np.float32(0))
    above = np.nextafter(mids.astype(np.float32), np.float32(1e9))
    edge = np.array([448, 449, 463.99, 464, 464.0001, 465, 480, 1e6, np.inf, -np.inf, -464, -465,
                     2.0 ** -10, 2.0 ** -10 * 1.0001, 3 * 2.0 ** -10, 0.0, -0.0, 1e-30], np.float32)
    x = np.concatenate([mids, -mids, below, above, edge]).astype(np.float32)
    assert np.array_equal(fp8.encode_e4m3(x), _torch_encode(x))
    # the rule itself: 464 ties down to 448, anything above is the NaN code
    assert fp8.encode_e4m3(np.float32(464.0)) == 0x7E
    assert fp8.encode_e4m3(np.float32(464.0001)) == 0x7F
    assert fp8.encode_e4m3(np.float32(2.0 ** -10)) == 0x00      # tie to even (zero)
    assert fp8.encode_e4m3(np.float32(3 * 2.0 ** -10)) == 0x02  # tie to even (2 * 2^-9)


def test_encode_random():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200000) * 120, rng.standard_normal(100000) * 0.01]).astype(np.float32)
    assert np.array_equal(fp8.encode_e4m3(x), _torch_encode(x))


def test_eager_quantize_matches_table():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4096, generator=g) * 2
    for s in (100 / 448, 1.6 / 448, 0.37):
        q = eager.quantize_e4m3(x, s).view(torch.uint8).numpy()
        ref = fp8.encode_e4m3((x / torch.tensor(s, dtype=torch.float32)).numpy())
        assert np.array_equal(q, ref)
        deq = eager.dequantize(eager.quantize_e4m3(x, s), s).numpy()
        assert np.array_equal(deq, (fp8.decode_e4m3(q).astype(np.float32) * np.float32(s)), equal_nan=True)
