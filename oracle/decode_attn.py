"""Ragged single-query attention over a static KV cache, numpy restatement (checker only).

Pinned by: tests/test_oracle_attn.py checks it against torch's scaled_dot_product_attention with an additive -inf
mask (the formulation of the reference's tests/test_math_kernels.py:85-98), against a per-row brute-force loop
that gathers keys by absolute position (an independent statement of the ring mapping), on the reference's ring /
left-pad edge vectors (tests/test_math_kernels.py:55-82), and against the C twin in uv_oracle.c.
"""
from __future__ import annotations

import numpy as np


def key_range(pos, starts, window: int):
    """Valid absolute key positions of each row are lo..pos inclusive, lo = max(starts, pos - window + 1, 0);
    decode_attn.py:197-203, 253-256."""
    p = np.asarray(pos, dtype=np.int64)
    lo = np.maximum(np.asarray(starts, dtype=np.int64), 0)
    if window > 0:
        lo = np.maximum(lo, p - window + 1)
    return lo, p


def decode_attention_ref(q, k_cache, v_cache, pos, starts, scale: float, *, window: int = 0, ring=None,
                         k_scale=None, v_scale=None, out_dtype=np.float32):
    """q (B, H, hd); caches (B, K, S, hd) float or int8 with (B, K, S) fp16 scales; returns (B, H, hd) fp32.
    Follows decode_attention_ref, ultraviolet/kernels/decode_attn.py:233-263: dequantise, map every slot to the
    absolute position it holds (ring: tpos = p - ((p - slot) mod S)), mask to lo..p, softmax(q.k*scale), weighted V."""
    q = np.asarray(q, dtype=np.float32)
    if q.ndim == 4:
        q = q.reshape(q.shape[0], q.shape[-2], q.shape[-1])
    B, H, hd = q.shape
    KH, S = k_cache.shape[1], k_cache.shape[2]
    G = H // KH
    if ring is None:
        ring = window > 0
    kf = np.asarray(k_cache, dtype=np.float32)
    vf = np.asarray(v_cache, dtype=np.float32)
    if k_cache.dtype == np.int8:
        kf = kf * np.asarray(k_scale, dtype=np.float32)[..., None]
        vf = vf * np.asarray(v_scale, dtype=np.float32)[..., None]
    slot = np.arange(S, dtype=np.int64)[None, :]
    lo, p = key_range(pos, starts, window)
    p, lo = p[:, None], lo[:, None]
    tpos = p - np.remainder(p - slot, S) if ring else np.broadcast_to(slot, (B, S))
    valid = (tpos >= lo) & (tpos <= p)
    qf = q.reshape(B, KH, G, hd)
    s = np.einsum("bkgd,bksd->bkgs", qf, kf, optimize=True) * np.float32(scale)
    s = np.where(valid[:, None, None, :], s, -np.inf).astype(np.float32)
    m = s.max(-1, keepdims=True)
    e = np.exp(s - m)
    w = e / e.sum(-1, keepdims=True)
    out = np.einsum("bkgs,bksd->bkgd", w.astype(np.float32), vf, optimize=True)
    return out.reshape(B, H, hd).astype(out_dtype)


def decode_attention_rows(q, k_cache, v_cache, pos, starts, scale: float, *, window: int = 0, ring=None,
                          k_scale=None, v_scale=None):
    """Brute-force statement of the same contract in float64: for every row walk the absolute positions
    lo..pos and read slot t (linear) or t % S (ring).  Independent of the slot->position inversion above."""
    q = np.asarray(q, dtype=np.float64)
    if q.ndim == 4:
        q = q.reshape(q.shape[0], q.shape[-2], q.shape[-1])
    B, H, hd = q.shape
    KH, S = k_cache.shape[1], k_cache.shape[2]
    G = H // KH
    if ring is None:
        ring = window > 0
    lo, p = key_range(pos, starts, window)
    out = np.zeros((B, H, hd), dtype=np.float64)
    for b in range(B):
        t = np.arange(lo[b], p[b] + 1)
        sl = t % S if ring else t
        for h in range(KH):
            k = np.asarray(k_cache[b, h, sl], dtype=np.float64)
            v = np.asarray(v_cache[b, h, sl], dtype=np.float64)
            if k_cache.dtype == np.int8:
                k = k * np.asarray(k_scale[b, h, sl], dtype=np.float64)[:, None]
                v = v * np.asarray(v_scale[b, h, sl], dtype=np.float64)[:, None]
            s = q[b, h * G:(h + 1) * G] @ k.T * scale
            w = np.exp(s - s.max(-1, keepdims=True))
            out[b, h * G:(h + 1) * G] = (w / w.sum(-1, keepdims=True)) @ v
    return out


def algorithmic_bytes(pos, starts, window: int, B: int, H: int, KH: int, hd: int, int8: bool = True) -> int:
    """HBM bytes the op must move: KH * (2*hd*esz + 4 if int8) per attended key + q and out (2 B each) + pos/starts."""
    lo, p = key_range(pos, starts, window)
    n = int((p - lo + 1).sum())
    per_key = 2 * hd + 4 if int8 else 4 * hd
    return KH * per_key * n + 4 * B * H * hd + 16 * B
