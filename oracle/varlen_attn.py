"""Packed (cu_seqlens) causal attention with an optional sliding window, numpy restatement (checker only).

Pinned by: tests/test_oracle_attn.py checks it against torch's scaled_dot_product_attention with a boolean mask
per segment (the definition the reference's own varlen test relies on, tests/test_perf_opt.py:40-61) on the
reference's segment lengths [300, 1000, 57, 700, 1] with window None / 256.
"""
from __future__ import annotations

import numpy as np


def varlen_attention_ref(q, k, v, cu_seqlens, scale: float, window=None):
    """q (N, H, hd), k/v (N, K, hd) packed along N; cu_seqlens (S+1,).  Query i of a segment sees keys j of the
    same segment with i - window < j <= i.  Follows varlen_attention_ref, kernels/varlen_attn.py:94-115."""
    q = np.asarray(q, dtype=np.float32)
    k = np.asarray(k, dtype=np.float32)
    v = np.asarray(v, dtype=np.float32)
    N, H, hd = q.shape
    K = k.shape[1]
    G = H // K
    out = np.zeros((N, H, hd), dtype=np.float32)
    cu = [int(c) for c in cu_seqlens]
    for a, b in zip(cu[:-1], cu[1:]):
        L = b - a
        if L == 0:
            continue
        i = np.arange(L)
        d = i[:, None] - i[None, :]
        m = d >= 0
        if window:
            m &= d < window
        for h in range(H):
            s = q[a:b, h] @ k[a:b, h // G].T * np.float32(scale)
            s = np.where(m, s, -np.inf)
            w = np.exp(s - s.max(-1, keepdims=True))
            out[a:b, h] = (w / w.sum(-1, keepdims=True)) @ v[a:b, h // G]
    return out
