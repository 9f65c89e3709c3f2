"""Pins oracle.fused_sample and oracle.philox: float64 softmax, the CDF-interval invariant, the reference's edge vectors
and chi-square test (tests/test_perf_fz.py:51-71, 96-119), Random123 known answers, and the C twin."""
import numpy as np
import pytest
import torch

from oracle import cbind, fused_sample, philox

SC = (23.0, 5.0, 7.5)


def _softcap64(x):
    return SC[0] / (1.0 + np.exp(-(np.asarray(x, np.float64) + SC[1]) / SC[2]))


@pytest.mark.parametrize("T", [1.0, 0.7])
def test_ref_sampler_distribution_and_logp(T):
    rng = np.random.default_rng(0)
    V, n = 256, 100_000
    x = (rng.standard_normal(V) * 6).astype(np.float32)
    z = _softcap64(x) / T
    p = np.exp(z - z.max())
    p /= p.sum()
    u = rng.random(n, dtype=np.float32)
    tok, lp = fused_sample.fused_sample_ref(np.broadcast_to(x, (n, V)), u, SC, T)
    cnt = np.bincount(tok, minlength=V).astype(np.float64)
    e = p * n
    big = e >= 5
    obs = np.concatenate([cnt[big], [cnt[~big].sum()]])
    ex = np.concatenate([e[big], [e[~big].sum()]])
    keep = ex > 0
    chi = ((obs[keep] - ex[keep]) ** 2 / ex[keep]).sum()
    pval = float(torch.special.gammaincc(torch.tensor((keep.sum() - 1) / 2, dtype=torch.float64), torch.tensor(chi / 2)))
    assert pval > 1e-3
    ref = (z - z.max() - np.log(np.exp(z - z.max()).sum()))[tok]
    assert np.abs(lp - ref).max() < 1e-4


def test_cdf_interval_invariant_and_c_twin():
    rng = np.random.default_rng(1)
    B, V = 64, 4096
    x = (rng.standard_normal((B, V)) * rng.random((B, 1)) * 8).astype(np.float16).astype(np.float32)
    u = rng.random(B, dtype=np.float32)
    for T in (1.0, 0.8):
        tok, lp = fused_sample.fused_sample_ref(x, u, SC, T)
        e = np.exp((_softcap64(x) - SC[0]) / T)
        cs = np.cumsum(e, -1)
        S = cs[:, -1]
        tgt = (1.0 - u.astype(np.float64)) * S
        hi = np.take_along_axis(cs, tok[:, None], 1)[:, 0]
        lo = hi - np.take_along_axis(e, tok[:, None], 1)[:, 0]
        assert ((tgt >= lo - 1e-5 * S) & (tgt <= hi + 1e-5 * S)).all()
        ctok, clp = cbind.fused_sample(x, u, SC, T)
        assert (ctok == tok).mean() > 0.95 and np.abs(clp - lp)[ctok == tok].max() < 1e-4


def test_edges_and_ok_predicate():
    """u -> 1 never picks a zero-mass prefix; u = 0 is clamped (tests/test_perf_fz.py:66-71); predicate (:74-77)."""
    x = np.full((2, 64), -1e4, np.float32)
    x[:, 40] = 10.0
    tok, _ = fused_sample.fused_sample_ref(x, np.array([0.0, 1.0 - 2 ** -24], np.float32), SC, 1.0)
    assert tok.max() < 64 and tok.min() >= 0
    assert fused_sample.fused_sample_ok(16384, SC, 1.0)
    assert not fused_sample.fused_sample_ok(16000, SC, 1.0)
    assert not fused_sample.fused_sample_ok(16384, SC, 0.1)
    assert list(fused_sample.greedy(np.array([[1.0, 3.0, 3.0, 2.0]]))) == [1]


def test_philox_known_answers():
    """Random123 kat_vectors for philox4x32-10."""
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
            (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for c, k, o in kat:
        assert tuple(int(v) for v in philox.philox4x32_10(c, k)) == o
        assert tuple(int(v) for v in cbind.philox(c, k)) == o


def test_request_uniform_mapping():
    u = philox.request_uniform(7, np.arange(1000), np.arange(1000) % 37)
    assert u.dtype == np.float32 and u.min() >= 0 and u.max() < 1 and abs(u.mean() - 0.5) < 0.05
    # counter layout: (tok_idx, req lo, req hi, "SAMP"), key = seed words
    r = philox.philox4x32_10((5, 9, 0, philox.DOMAIN_SAMPLE), (7, 0))
    assert philox.request_uniform(7, 9, 5) == np.float32((int(r[0]) >> 8) * 2.0 ** -24)
    assert philox.request_uniform(7, 9, 5) != philox.request_uniform(7, 9, 5, philox.DOMAIN_RETIRE)
