"""Packed (cu_seqlens) causal attention with an optional sliding window, numpy restatement (checker only).

Pinned by: tests/test_oracle_attn.py checks it against torch's scaled_dot_product_attention with a boolean mask
per segment (the definition the reference's own varlen test relies on, tests/test_perf_opt.py:40-61) on the
reference's segment lengths [300, 1000, 57, 700, 1] with window None / 256.  varlen_attention_grad_ref (the backward,
kernels/varlen_attn.py:56-66) is pinned there by central finite differences of the forward restatement on tiny inputs in
float64 and by torch autograd through a masked-softmax formulation.
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


def varlen_attention_grad_ref(q, k, v, go, cu_seqlens, scale: float, window=None):
    """(dq, dk, dv) of sum(out * go) for out = varlen_attention_ref(q, k, v, ...), in float64: what the reference's
    backward returns (mathk::varlen_attn_bwd, kernels/varlen_attn.py:56-66: the memory-efficient attention backward on
    K / V expanded to the query heads, their gradients summed back over each group)."""
    q, k, v, go = (np.asarray(x, dtype=np.float64) for x in (q, k, v, go))
    N, H, hd = q.shape
    K = k.shape[1]
    G = H // K
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
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
            kh = h // G
            s = np.where(m, q[a:b, h] @ k[a:b, kh].T * scale, -np.inf)
            p = np.exp(s - s.max(-1, keepdims=True))
            p /= p.sum(-1, keepdims=True)
            o = p @ v[a:b, kh]
            dp = go[a:b, h] @ v[a:b, kh].T
            ds = p * (dp - (go[a:b, h] * o).sum(-1, keepdims=True))
            dq[a:b, h] = ds @ k[a:b, kh] * scale
            dk[a:b, kh] += ds.T @ q[a:b, h] * scale
            dv[a:b, kh] += p.T @ go[a:b, h]
    return dq, dk, dv
