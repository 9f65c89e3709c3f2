"""Softcap + inverse-CDF categorical draw + behaviour log-prob, numpy restatement (checker only).

Pinned by: tests/test_oracle_sample.py checks the closed form against float64 log_softmax (|logp - ref| < 1e-4,
tests/test_perf_fz.py:51-63), the CDF-interval invariant (:96-119), the edge vectors (:66-71), a chi-square draw
test and the C twin in uv_oracle.c.
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
