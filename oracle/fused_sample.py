"""Softcap + inverse-CDF categorical draw + behaviour log-prob, numpy restatement (checker only).

Pinned by: tests/test_oracle_sample.py checks the closed form against float64 log_softmax (|logp - ref| < 1e-4,
tests/test_perf_fz.py:51-63), the CDF-interval invariant (:96-119), the edge vectors (:66-71), a chi-square draw
test and the C twin in uv_oracle.c.  The truncated sampler (filter_mask, sample_filtered_ref) is pinned by the properties
that define sample()'s top-k / nucleus sets (top set by value, exactly k members, minimal nucleus of mass >= top_p, ties of
the cut kept), brute-force enumeration on tiny vocabularies and a chi-square of its draws.
"""
from __future__ import annotations

import numpy as np


def softcap(x, sc=(23.0, 5.0, 7.5)):
    """a * sigmoid((x + b) / c) in fp32; ultraviolet/model.py:824-827."""
    a, b, c = (np.float32(v) for v in sc)
    t = (np.asarray(x, dtype=np.float32) + b) / c
    return (a / (np.float32(1.0) + np.exp(-t))).astype(np.float32)


def fused_sample_ref(x, u, sc=(23.0, 5.0, 7.5), temperature: float = 1.0):
    """x (B, V) raw head output, u (B,) uniforms in [0, 1) -> (tok int64 (B,), logp fp32 (B,)).
    Follows fused_sample_ref, ultraviolet/kernels/fused_sample.py:79-91: e = exp((z - a)/T) with z the softcapped
    logit (bounded by a, so no max pass), flat fp32 cumsum, token = first index whose cumsum >= (1 - u) * S
    (searchsorted, left), clamped to V - 1; logp = (z_tok - a)/T - log S."""
    a = np.float32(sc[0])
    T = np.float32(temperature)
    z = softcap(x, sc)
    e = np.exp((z - a) / T).astype(np.float32)
    cs = np.cumsum(e, axis=-1, dtype=np.float32)
    S = cs[:, -1]
    target = (np.float32(1.0) - np.asarray(u, dtype=np.float32)) * S
    tok = np.array([np.searchsorted(cs[i], target[i], side="left") for i in range(cs.shape[0])], dtype=np.int64)
    tok = np.minimum(tok, x.shape[1] - 1)
    zt = np.take_along_axis(z, tok[:, None], 1)[:, 0]
    lp = (zt - a) / T - np.log(S)
    return tok, lp.astype(np.float32)


def fused_sample_ok(V: int, sc, temperature: float, block: int = 1024) -> bool:
    """Shape/temperature predicate of ultraviolet/kernels/fused_sample.py:61-65 (device checks left out)."""
    return V % block == 0 and V // block <= 64 and temperature > 0 and float(sc[0]) / temperature <= 80.0


def greedy(logits) -> np.ndarray:
    """T <= 0 branch of sample(): argmax, first maximal index; ultraviolet/model.py:1198-1199."""
    return np.argmax(np.asarray(logits), axis=-1).astype(np.int64)


def filter_mask(z, top_k: int = 0, top_p: float = 1.0) -> np.ndarray:
    """Which tokens sample() keeps (ultraviolet/model.py:1200-1209), z (V,) = logits / T: with top_k, the tokens whose
    value is at least the k-th largest (`z < kth` is masked); with top_p < 1, of those the sorted prefix whose preceding
    softmax mass is below top_p (`(ps.cumsum(-1) - ps) < top_p`), cut at the smallest kept VALUE (`z < cut` is masked, so
    ties of the cut value are all kept).  float64."""
    z = np.asarray(z, dtype=np.float64).copy()
    V = z.shape[0]
    keep = np.ones(V, dtype=bool)
    if top_k and top_k < V:
        kth = np.sort(z)[::-1][top_k - 1]
        keep &= z >= kth
    if top_p < 1.0:
        zm = np.where(keep, z, -np.inf)
        zs = np.sort(zm)[::-1]
        ps = np.exp(zs - zs[0])
        ps /= ps.sum()
        kept_sorted = (np.cumsum(ps) - ps) < top_p
        kept_sorted[0] = True   # the first token is always kept (cumsum - p is 0 there; written out for top_p <= 0)
        cut = zs[kept_sorted].min()
        keep &= zm >= cut
    return keep


def sample_filtered_ref(x, u, sc=(23.0, 5.0, 7.5), temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0):
    """Truncated draw by inverse CDF in index order over the kept tokens (the distribution sample() draws from with its
    Gumbel-max, model.py:1210-1211), float64; logp of the untruncated softmax (model.py:1161-1169).
    x (B, V), u (B,) -> tok (B,), logp (B,), keep (B, V) bool."""
    x = np.asarray(x, dtype=np.float64)
    a, b, c = (float(v) for v in sc)
    z = a / (1.0 + np.exp(-(x + b) / c)) / temperature
    B, V = z.shape
    tok = np.zeros(B, dtype=np.int64)
    lp = np.zeros(B)
    keep = np.zeros((B, V), dtype=bool)
    for i in range(B):
        keep[i] = filter_mask(z[i], top_k, top_p)
        e = np.where(keep[i], np.exp(z[i] - z[i].max()), 0.0)
        cs = np.cumsum(e)
        t = min(int(np.searchsorted(cs, (1.0 - float(u[i])) * cs[-1], side="left")), V - 1)
        while not keep[i, t]:
            t -= 1
        tok[i] = t
        lp[i] = z[i, t] - (z[i].max() + np.log(np.exp(z[i] - z[i].max()).sum()))
    return tok, lp, keep
