"""Pins oracle.kv_quant (and its C twin) without the reference: exact rational arithmetic, the reference's own test
vectors (tests/test_math_kernels.py:115-128) and brute force on index math."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import cbind, kv_quant


def _round_to(fr: Fraction, p: int, emin: int) -> Fraction:
    """Round a non-negative rational to the nearest value with p significand bits and minimum exponent emin
    (subnormals included), ties to even: IEEE round-to-nearest-even done in integers."""
    if fr == 0:
        return Fraction(0)
    e = fr.numerator.bit_length() - fr.denominator.bit_length()
    if Fraction(2) ** e > fr:
        e -= 1
    e = max(e, emin)
    q = Fraction(2) ** (e - p + 1)   # spacing
    n = fr / q
    fl = n.numerator // n.denominator
    rem = n - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return fl * q


def _quant_exact(row):
    """quantize_kv in exact arithmetic: fp32 division, fp16 RNE, fp32 division, round-half-even, clamp."""
    xs = [Fraction(float(v)) for v in row]
    amax = max(abs(v) for v in xs)
    s32 = _round_to(amax / 127, 24, -126)
    s16 = _round_to(s32, 11, -14)
    if s16 >= Fraction(65520):
        return None, None  # fp16 overflow: inf scale, not exercised here
    sf = max(s16, _round_to(Fraction(1, 10 ** 30), 24, -126))
    out = []
    for v in xs:
        qf = _round_to(abs(v) / sf, 24, -126)          # fp32 quotient
        fl = qf.numerator // qf.denominator
        rem = qf - fl
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
            fl += 1
        fl = min(fl, 127)
        out.append(-fl if v < 0 else fl)
    return out, float(s16)


@pytest.mark.parametrize("dtype", [np.float16, np.float32, "bf16"])
def test_quantizer_matches_exact_rational_arithmetic(dtype):
    rng = np.random.default_rng(0)
    rows = []
    for scale in (1.0, 3.0, 1e-3, 1e-6, 2e-8, 300.0):
        x = (rng.standard_normal((40, 16)) * scale).astype(np.float32)
        if dtype == "bf16":
            x = (x.view(np.uint32) & 0xFFFF0000).view(np.float32)
        elif dtype == np.float16:
            x = x.astype(np.float16).astype(np.float32)
        rows.append(x)
    x = np.concatenate(rows)
    x[3] = 0.0
    x[5, 2] = x[5].max() * 0 + 127.0 * 0.0037  # hits exact half-way codes for some columns
    x[7] = np.arange(16) * 0.5 - 3.75          # exact ties x/s = k + 0.5
    q, s = kv_quant.quantize_kv(x)
    for r in range(x.shape[0]):
        eq, es = _quant_exact(x[r])
        assert list(q[r]) == eq, r
        assert float(s[r]) == es, r
    cq, cs = cbind.quantize_rows(x)
    assert np.array_equal(cq, q) and np.array_equal(cs.view(np.uint16), s.view(np.uint16))


def test_quantizer_reference_vectors():
    """tests/test_math_kernels.py:115-121: zero row -> zeros; |deq - x| <= s/2 (+1e-3)."""
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((64, 3, 128)) * 3).astype(np.float16)
    x[0, 0] = 0
    q, s = kv_quant.quantize_kv(x)
    err = np.abs(kv_quant.dequantize_kv(q, s) - x.astype(np.float32))
    assert err.max() <= (s.astype(np.float32)[..., None] * 0.5 + 1e-3).max()
    assert (q[0, 0] == 0).all() and s[0, 0] == 0
    assert np.abs(q).max() <= 127


def test_scale_underflow_and_clamp():
    """A scale that underflows fp16 gives codes +-127 with s = 0 (the 1e-30 floor); fp16 rounding of the scale moves
    absmax / s by at most 2^-11 around 127, so the top code is always 127 and the clamp is what caps it when the scale
    was rounded down."""
    x = np.full((1, 8), 1e-9, np.float32)
    x[0, 1] = -1e-9
    q, s = kv_quant.quantize_kv(x)
    assert s[0] == 0 and q[0, 0] == 127 and q[0, 1] == -127
    rng = np.random.default_rng(2)
    x = rng.standard_normal((4000, 64)).astype(np.float32)
    q, s = kv_quant.quantize_kv(x)
    assert (np.abs(q).max(-1) == 127).all()
    ratio = np.abs(x).max(-1) / s.astype(np.float32)
    assert (ratio > 127.0).any() and (ratio < 127.0).any() and np.abs(ratio - 127).max() < 127 * 2.0 ** -10


def test_flat_index_write_reference_vector():
    """tests/test_math_kernels.py:122-128: idx = [3, 31, 32, 55] on a (4, 1, 16, 128) cache."""
    rng = np.random.default_rng(3)
    cache = np.zeros((4, 1, 16, 128), np.int8)
    sc = np.zeros((4, 1, 16), np.float16)
    idx = np.array([0 * 16 + 3, 1 * 16 + 15, 2 * 16 + 0, 3 * 16 + 7])
    assert list(idx) == [3, 31, 32, 55]
    xv = rng.standard_normal((4, 128)).astype(np.float16)
    kv_quant.kv_write(cache, sc, idx, xv)
    q, s = kv_quant.quantize_kv(xv)
    for r, (b, slot) in enumerate([(0, 3), (1, 15), (2, 0), (3, 7)]):
        assert np.array_equal(cache[b, 0, slot], q[r]) and sc[b, 0, slot] == s[r]
    assert np.count_nonzero(sc) == 4
    back = kv_quant.dequantize_kv(cache.reshape(-1, 128)[idx], sc.reshape(-1)[idx])
    np.testing.assert_allclose(back, xv.astype(np.float32), atol=0.03, rtol=0.03)


def test_decode_and_prefill_indices_brute_force():
    """(b*K + h)*S + pos and ring pos % S (fast_decode.py:291-294); ring survivors pos >= T - S (:175-177)."""
    B, K, S = 5, 2, 8
    pos = np.array([0, 7, 8, 19, 3])
    for ring in (False, True):
        ix = kv_quant.decode_flat_index(pos, K, S, ring)
        exp = [(b * K + h) * S + (pos[b] % S if ring else pos[b]) for b in range(B) for h in range(K)]
        assert list(ix) == exp
    T = 21
    p = np.arange(T)
    bk = np.full((T, 1), 3)
    sel, ix = kv_quant.prefill_write_index(p, bk, S, T, is_global=False)
    assert list(sel) == list(range(T - S, T))
    assert sorted(ix % S) == list(range(S))           # every ring slot written exactly once
    assert list(ix) == [3 * S + (t % S) for t in range(T - S, T)]
    sel, ix = kv_quant.prefill_write_index(p, bk, 64, T, is_global=True)
    assert sel is None and list(ix) == [3 * 64 + t for t in range(T)]


def test_kv_write_rows_equals_per_token_writes():
    rng = np.random.default_rng(4)
    B, K, S, hd, T = 6, 2, 16, 32, 21
    new = rng.standard_normal((3, K, T, hd)).astype(np.float32)
    rows = np.array([4, 0, 3])
    lo = T - S
    c1, s1 = np.zeros((B, K, S, hd), np.int8), np.zeros((B, K, S), np.float16)
    kv_quant.kv_write_rows(c1, s1, new[:, :, lo:], np.arange(lo, T) % S, rows)
    c2, s2 = np.zeros_like(c1), np.zeros_like(s1)
    for i, r in enumerate(rows):
        for h in range(K):
            for t in range(lo, T):
                kv_quant.kv_write(c2, s2, np.array([(r * K + h) * S + t % S]), new[i, h, t][None])
    assert np.array_equal(c1, c2) and np.array_equal(s1.view(np.uint16), s2.view(np.uint16))
