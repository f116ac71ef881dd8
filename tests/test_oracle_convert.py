"""Pins the oracle's 16-bit float conversions against numpy (binary16) and torch (bfloat16)."""
import numpy as np
import torch

from helpers import BF16, FP16, exact_round16
from fractions import Fraction
from oracle import oracle as orc


def test_f16_to_f32_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = orc.from_bits(bits, FP16)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def _edge_floats(rng):
    vals = [0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e30, -1e30, 2.0 ** -24, 2.0 ** -25,
            2.0 ** -25 * 1.0000001, 2.0 ** -14, 2.0 ** -14 * 0.9999, 6.1e-5, 1.0009765625, 1.00048828125,
            1.00146484375, 3.0e-8, 2.98e-8, float("inf"), float("-inf")]
    # every tie between adjacent binary16 values in a few binades, and their float32 neighbours
    for e in (-16, -15, -14, -1, 0, 10, 15):
        base = np.float32(2.0 ** e)
        step = np.float32(2.0 ** (e - 10))
        for k in range(0, 12):
            t = np.float32(base + step * (k + 0.5))
            vals += [t, np.nextafter(t, np.float32(np.inf)), np.nextafter(t, np.float32(-np.inf))]
    r = rng.standard_normal(200000).astype(np.float32) * (10.0 ** rng.uniform(-9, 6, 200000)).astype(np.float32)
    u = rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    u = u[np.isfinite(u)]
    return np.concatenate([np.array(vals, np.float32), r, u])


def test_f32_to_f16_vs_numpy():
    x = _edge_floats(np.random.default_rng(1))
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = orc.to_bits(x, FP16)
    assert np.array_equal(got, want)


def test_f32_to_f16_nan():
    got = orc.to_bits(np.array([np.nan], np.float32), FP16)
    assert np.isnan(got.view(np.float16)[0])


def test_bf16_vs_torch():
    x = _edge_floats(np.random.default_rng(2))
    t = torch.from_numpy(x.copy())
    want = t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = orc.to_bits(x, BF16)
    assert np.array_equal(got, want)
    bits = np.arange(65536, dtype=np.uint16)
    back = orc.from_bits(bits, BF16)
    want_back = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).to(torch.float32).numpy()
    nan = np.isnan(want_back)
    assert np.array_equal(back[~nan].view(np.uint32), want_back[~nan].view(np.uint32))
    assert np.all(np.isnan(back[nan]))


def test_exact_round_helper_agrees_with_numpy():
    # the exact-rational rounding used by the arithmetic pins must itself be right
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(3000) * 10.0 ** rng.uniform(-6, 4, 3000)).astype(np.float64)
    for v in x:
        want = int(np.float16(v).view(np.uint16)) if abs(v) < 65504 else None
        if want is None:
            continue
        assert exact_round16(Fraction(float(v)), FP16) == want
        tb = torch.tensor(float(np.float32(v)), dtype=torch.float32).to(torch.bfloat16).view(torch.int16).item() & 0xffff
        assert exact_round16(Fraction(float(np.float32(v))), BF16) == tb
