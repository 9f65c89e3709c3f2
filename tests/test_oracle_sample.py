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


# ---- truncated sampling (top-k / nucleus): the oracle's filter against what defines it
def test_filter_mask_is_a_top_set_with_k_members_and_minimal_nucleus():
    """Properties that fix sample()'s truncation (ultraviolet/model.py:1200-1209) without restating it: the kept set is a
    top set by value; top-k keeps exactly k tokens when values are distinct; the nucleus has mass >= top_p and is minimal
    (dropping its smallest member leaves less than top_p); the most likely token always survives; no filter keeps all."""
    from oracle.fused_sample import filter_mask
    rng = np.random.default_rng(0)
    for V, k, p in [(64, 5, 1.0), (64, 0, 0.7), (512, 40, 0.9), (512, 3, 0.2), (33, 32, 0.999), (128, 1, 0.5), (128, 0, 1e-9)]:
        z = rng.normal(size=V) * 3
        keep = filter_mask(z, k, p)
        assert keep[np.argmax(z)]
        assert z[keep].min() > z[~keep].max() if (~keep).any() else True
        pr = np.exp(z - z.max()); pr /= pr.sum()
        if k and p >= 1.0:
            assert keep.sum() == k
        if p < 1.0:
            base = np.ones(V, bool) if not k else filter_mask(z, k, 1.0)
            q = np.where(base, pr, 0.0); q /= q.sum()          # the nucleus is taken inside the top-k set, renormalised
            m = q[keep].sum()
            assert m >= p - 1e-12 or keep.sum() == base.sum()
            assert m - q[keep].min() < p                        # minimal: without its smallest member the mass is short
    assert filter_mask(rng.normal(size=50), 0, 1.0).all()


def test_filter_mask_keeps_ties_of_the_cut_value():
    from oracle.fused_sample import filter_mask
    z = np.array([3.0, 1.0, 2.0, 2.0, 2.0, 0.0, -1.0])
    assert filter_mask(z, 2, 1.0).tolist() == [True, False, True, True, True, False, False]      # k-th value 2.0: all three 2.0s stay
    pr = np.exp(z - 3.0); pr /= pr.sum()
    p = pr[0] + 1e-6                                                                             # crossing inside the tie group
    assert filter_mask(z, 0, p).tolist() == [True, False, True, True, True, False, False]


def test_filter_mask_brute_force_small():
    """Every subset rule checked by enumeration on tiny V: the nucleus equals the shortest sorted prefix whose mass reaches
    top_p, found by trying every prefix length."""
    from oracle.fused_sample import filter_mask
    rng = np.random.default_rng(3)
    for _ in range(200):
        V = int(rng.integers(2, 9))
        z = rng.normal(size=V) * 2
        p = float(rng.uniform(0.05, 0.99))
        order = np.argsort(-z)
        pr = np.exp(z - z.max()); pr /= pr.sum()
        n = next(n for n in range(1, V + 1) if pr[order[:n]].sum() >= p or n == V)
        want = np.zeros(V, bool); want[order[:n]] = True
        assert (filter_mask(z, 0, p) == want).all()


def test_sample_filtered_ref_draws_only_kept_tokens_in_proportion():
    from oracle.fused_sample import sample_filtered_ref, fused_sample_ref
    rng = np.random.default_rng(5)
    x = rng.normal(size=(1, 32)).astype(np.float32) * 4
    n = 4000
    u = rng.random(n)
    tok, lp, keep = sample_filtered_ref(np.repeat(x, n, 0), u, temperature=0.8, top_k=6, top_p=0.9)
    assert keep[0, tok].all()
    z = 23.0 / (1.0 + np.exp(-(x[0].astype(np.float64) + 5.0) / 7.5)) / 0.8
    q = np.where(keep[0], np.exp(z - z.max()), 0.0); q /= q.sum()
    cnt = np.bincount(tok, minlength=32)
    chi = ((cnt - n * q) ** 2 / np.maximum(n * q, 1e-12))[q > 0].sum()
    assert chi < 40, chi                                    # <= 5 degrees of freedom
    # log-prob is the untruncated one; no filter reproduces the plain sampler's token
    t0, l0 = fused_sample_ref(np.repeat(x, 16, 0), u[:16].astype(np.float32), temperature=0.8)
    t1, l1, _ = sample_filtered_ref(np.repeat(x, 16, 0), u[:16], temperature=0.8)
    assert (t0 == t1).all() and np.abs(l0 - l1).max() < 1e-5
    full = z - (z.max() + np.log(np.exp(z - z.max()).sum()))
    assert np.abs(lp - full[tok]).max() < 1e-12
