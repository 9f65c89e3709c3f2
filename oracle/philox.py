"""Philox4x32-10 counter-based RNG and the engine's seed mapping, numpy restatement (checker only).

The reference has no RNG code of its own (it calls torch.rand: ultraviolet/perf.py:595, model.py:1210), so the
engine defines the stream: one uniform per (request id, token index) so that a request's draws do not depend on
which slot it occupies or when it was admitted.

Pinned by: the three Random123 known-answer vectors for philox4x32-10 (tests/test_oracle_philox.py) and the C twin.
"""
from __future__ import annotations

import numpy as np

M0, M1 = 0xD2511F53, 0xCD9E8D57
W0, W1 = 0x9E3779B9, 0xBB67AE85
MASK = 0xFFFFFFFF
DOMAIN_SAMPLE = 0x53414D50   # "SAMP": uniforms consumed by the token sampler
DOMAIN_RETIRE = 0x52455452   # "RETR": Bernoulli draws of the synthetic retire-with-probability-p workload


def philox4x32_10(ctr, key):
    """ctr: 4 uint32 (array-like, broadcastable leading dims as (..., 4)); key: 2 uint32 (..., 2)."""
    c = np.array(ctr, dtype=np.uint64) & MASK
    k = np.array(key, dtype=np.uint64) & MASK
    c0, c1, c2, c3 = (c[..., i].copy() for i in range(4))
    k0, k1 = k[..., 0].copy(), k[..., 1].copy()
    for _ in range(10):
        p0 = M0 * c0
        p1 = M1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK
        c0, c1, c2, c3 = (hi1 ^ c1 ^ k0) & MASK, lo1, (hi0 ^ c3 ^ k1) & MASK, lo0
        k0 = (k0 + W0) & MASK
        k1 = (k1 + W1) & MASK
    return np.stack([c0, c1, c2, c3], -1).astype(np.uint32)


def uniform_from_u32(x) -> np.ndarray:
    """Top 24 bits -> fp32 in [0, 1) (exact)."""
    return ((np.asarray(x, dtype=np.uint32) >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24))


def request_uniform(seed: int, req_id, tok_idx, domain: int = DOMAIN_SAMPLE) -> np.ndarray:
    """u for (request id, token index): counter = (tok_idx, req_id lo, req_id hi, domain), key = seed lo/hi;
    first output word."""
    req = np.asarray(req_id, dtype=np.uint64)
    tok = np.asarray(tok_idx, dtype=np.uint64)
    req, tok = np.broadcast_arrays(req, tok)
    ctr = np.stack([tok & MASK, req & MASK, req >> np.uint64(32), np.full(req.shape, domain, dtype=np.uint64)], -1)
    key = np.broadcast_to(np.array([seed & MASK, (seed >> 32) & MASK], dtype=np.uint64), req.shape + (2,))
    return uniform_from_u32(philox4x32_10(ctr, key)[..., 0])
