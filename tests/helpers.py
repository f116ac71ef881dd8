"""Shared test helpers: bit-pattern conversions, random paged pools, exact rounding."""
from __future__ import annotations

from fractions import Fraction

import numpy as np

from oracle import oracle as orc

FP16, BF16 = orc.FP16, orc.BF16


def bits_of(a: np.ndarray, dtype: int) -> np.ndarray:
    """fp32 values -> 16-bit patterns via numpy/torch-independent path of the oracle."""
    return orc.to_bits(a, dtype)


def f32_of(b: np.ndarray, dtype: int) -> np.ndarray:
    return orc.from_bits(b, dtype)


def torch_to_bits(t):
    import torch
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def bits_to_torch(b: np.ndarray, dtype: int, device="cpu"):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(b).view(np.int16).copy())
    return t.view(torch.float16 if dtype == FP16 else torch.bfloat16).to(device)


def ulp16(v: np.ndarray, dtype: int) -> np.ndarray:
    """Spacing of the 16-bit type at |v| (normal range)."""
    mant = 10 if dtype == FP16 else 7
    emin = -14 if dtype == FP16 else -126
    a = np.abs(v).astype(np.float64)
    e = np.floor(np.log2(np.maximum(a, 2.0 ** emin)))
    return 2.0 ** (e - mant)


class PagedPool:
    """Numpy model of the paged pool for one (layer, projection): the layout of include/mlora.h."""

    def __init__(self, rng, ranks, hin, hout, page_rows=8, dtype=FP16, std=0.02, extra_pages=3, shuffle=True,
                 max_pages=None, integer=False):
        ranks = np.asarray(ranks, np.int32)
        self.ranks = ranks
        self.n = len(ranks)
        self.page_rows = page_rows
        self.dtype = dtype
        need = [(int(r) + page_rows - 1) // page_rows for r in ranks]
        self.max_pages = max_pages or max(1, max(need))
        self.n_pages = sum(need) + extra_pages
        order = rng.permutation(self.n_pages) if shuffle else np.arange(self.n_pages)
        self.page_tbl = np.full((self.n, self.max_pages), -1, np.int32)
        pos = 0
        for i, k in enumerate(need):
            self.page_tbl[i, :k] = order[pos:pos + k]
            pos += k
        n_rows = self.n_pages * page_rows
        if integer:
            a = rng.integers(-1, 2, size=(n_rows, hin)).astype(np.float32)
            b = rng.integers(-1, 2, size=(n_rows, hout)).astype(np.float32)
        else:
            a = (rng.standard_normal((n_rows, hin)) * std).astype(np.float32)
            b = (rng.standard_normal((n_rows, hout)) * std).astype(np.float32)
        self.a_rows = bits_of(a, dtype)
        self.b_rows = bits_of(b, dtype)
        self.scaling = (32.0 / np.maximum(ranks, 1)).astype(np.float32)
        self.hin, self.hout = hin, hout

    def rows(self, i):
        j = np.arange(int(self.ranks[i]))
        return self.page_tbl[i, j // self.page_rows].astype(np.int64) * self.page_rows + j % self.page_rows

    def A(self, i):
        """A_i as float64 [Hin, r]."""
        return f32_of(self.a_rows[self.rows(i)], self.dtype).astype(np.float64).T

    def B(self, i):
        """B_i as float64 [r, Hout]."""
        return f32_of(self.b_rows[self.rows(i)], self.dtype).astype(np.float64)


def exact_round16(fr: Fraction, dtype: int) -> int:
    """Correctly rounded (nearest even) 16-bit pattern of an exact rational; finite, in range."""
    if fr == 0:
        return 0
    sign = 0x8000 if fr < 0 else 0
    a = abs(fr)
    mant = 10 if dtype == FP16 else 7
    bias = 15 if dtype == FP16 else 127
    emin = 1 - bias
    # exponent e with 2^e <= a < 2^(e+1)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, emin)
    q = a / (Fraction(2) ** (e - mant))          # significand in units of one ulp
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (n & 1)):
        n += 1
    if n >= (2 << mant):                         # carried into the next binade
        n >>= 1
        e += 1
    if n < (1 << mant):                          # subnormal
        return sign | n
    return sign | ((e + bias) << mant) | (n - (1 << mant))
