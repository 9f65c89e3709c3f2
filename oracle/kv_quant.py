"""int8 KV quantizer and cache writes, numpy restatement (checker only; see oracle/__init__.py).

Pinned by: the closed form below is fully determined by IEEE arithmetic (fp32 divide, fp16 round-to-nearest-even,
round-half-even); tests/test_oracle_quant.py checks it against exhaustive sweeps over all fp16/bf16 bit patterns
computed a second, independent way (integer arithmetic on the scale, fractions.Fraction for the division), the
reference's own test vectors (zero row, error bound s/2, flat-index write at idx [3, 31, 32, 55]:
tests/test_math_kernels.py:115-128) and the C twin in uv_oracle.c.
"""
from __future__ import annotations

import numpy as np


def quantize_kv(x: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """x (..., hd) float -> (int8 (..., hd), fp16 scale (...)).  Follows ultraviolet/kernels/kv_quant.py:12-19:
    s16 = fp16(absmax / 127); the row is divided by the fp16-ROUNDED scale (floored at 1e-30 so zero rows give
    q = 0), rounded half-to-even and clamped to +-127."""
    xf = np.asarray(x, dtype=np.float32)
    s16 = (np.abs(xf).max(axis=-1) / np.float32(127.0)).astype(np.float16)
    sf = np.maximum(s16.astype(np.float32), np.float32(1e-30))
    with np.errstate(over="ignore", invalid="ignore"):
        q = np.rint(xf / sf[..., None])
    q = np.clip(q, -127.0, 127.0).astype(np.int8)
    return q, s16


def dequantize_kv(q: np.ndarray, s: np.ndarray, dtype=np.float32) -> np.ndarray:
    """ultraviolet/kernels/kv_quant.py:22-23."""
    return (q.astype(np.float32) * s.astype(np.float32)[..., None]).astype(dtype)


def kv_write(cache: np.ndarray, scale: np.ndarray | None, flat_idx: np.ndarray, x: np.ndarray) -> None:
    """Decode-time append of one token per (row, kv head); ultraviolet/kernels/kv_quant.py:26-36.
    cache (B, K, S, hd) int8 (or float when scale is None); flat_idx (B*K,) = (b*K + h)*S + slot; in place."""
    hd = cache.shape[-1]
    x = np.asarray(x).reshape(-1, hd)
    flat = cache.reshape(-1, hd)
    assert flat.base is not None or flat is cache, "cache must be contiguous"
    if scale is None:
        flat[flat_idx] = x.astype(cache.dtype)
    else:
        q, s = quantize_kv(x)
        flat[flat_idx] = q
        scale.reshape(-1)[flat_idx] = s


def kv_write_rows(cache: np.ndarray, scale: np.ndarray | None, new: np.ndarray, slots, rows=None) -> None:
    """Prefill-time write: new (n, K, T', hd) goes to cache[rows][:, :, slots]; kv_quant.py:39-54."""
    vals = [(cache, new.astype(cache.dtype))] if scale is None else list(zip((cache, scale), quantize_kv(new)))
    for dst, src in vals:
        if rows is None:
            dst[:, :, slots] = src
        else:
            blk = dst[rows]
            blk[:, :, slots] = src
            dst[rows] = blk


def decode_flat_index(pos: np.ndarray, KH: int, S: int, ring: bool) -> np.ndarray:
    """Flat write index of the token at absolute position pos[b] for every (row, kv head):
    (b*K + h)*S + pos (linear cache) or (b*K + h)*S + pos % S (ring); fast_decode.py:291-294."""
    B = pos.shape[0]
    bk = np.arange(B, dtype=np.int64)[:, None] * KH + np.arange(KH, dtype=np.int64)[None, :]
    slot = pos.astype(np.int64)[:, None]
    if ring:
        slot = np.remainder(slot, S)
    return (bk * S + slot).reshape(-1)


def prefill_write_index(pos: np.ndarray, bk: np.ndarray, S: int, T: int, is_global: bool):
    """Packed-prefill cache indices; fast_decode.py:166-181.  pos (N,) left-padded position of every packed token,
    bk (N, K) cache row (row*K + h) of every token.  Returns (sel, ix): sel = packed-token subset that is written
    (None = all; ring layers keep only pos >= T - S) and ix (len(sel)*K,) flat indices bk*S + slot."""
    if is_global:
        return None, (bk * S + pos[:, None]).reshape(-1)
    sel = np.nonzero(pos >= T - S)[0]
    slot = pos[sel] % S
    return sel, (bk[sel] * S + slot[:, None]).reshape(-1)
