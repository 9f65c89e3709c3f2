"""Pins oracle.decode_attn and oracle.varlen_attn: torch SDPA with additive / boolean masks (the formulation the
reference's own tests rely on), a per-row brute force in float64, the reference's edge vectors, and the C twin."""
import numpy as np
import pytest
import torch

from oracle import cbind, decode_attn, varlen_attn
from util import attn_case, to_np


def _sdpa(q, k, v, ks, vs, pos, starts, scale, window, ring):
    """Dense masked attention through torch SDPA (tests/test_math_kernels.py:85-98 formulation), float64."""
    B, H, hd = q.shape
    KH, S = k.shape[1], k.shape[2]
    G = H // KH
    kf, vf = k.double(), v.double()
    if ks is not None:
        kf, vf = kf * ks.double()[..., None], vf * vs.double()[..., None]
    slot = torch.arange(S)[None]
    p = pos[:, None]
    lo = starts[:, None].clamp(min=0)
    if window:
        lo = torch.maximum(lo, p - window + 1)
    valid = torch.zeros(B, S, dtype=torch.bool)
    for b in range(B):  # position held by each slot, stated by walking positions (independent of the oracle's formula)
        for t in range(int(lo[b]), int(p[b]) + 1):
            valid[b, t % S if ring else t] = True
    bias = torch.zeros(B, S, dtype=torch.float64).masked_fill(~valid, float("-inf"))[:, None, None].expand(B, KH, G, S)
    z = torch.nn.functional.scaled_dot_product_attention(q.double().view(B, KH, G, hd), kf, vf, attn_mask=bias, scale=scale)
    return z.reshape(B, H, hd).numpy()


@pytest.mark.parametrize("int8", [False, True])
@pytest.mark.parametrize("B,KH,G,hd", [(3, 1, 4, 128), (5, 2, 4, 64), (9, 1, 8, 64), (4, 2, 2, 16)])
def test_global_ragged_vs_sdpa_and_rows(int8, B, KH, G, hd):
    S = 300
    q, k, v, ks, vs = attn_case(B, KH, G, hd, S, int8)
    g = torch.Generator().manual_seed(1)
    pos = torch.randint(0, S, (B,), generator=g)
    pos[0] = S - 1
    starts = (torch.rand(B, generator=g) * (pos + 1).float()).long()
    starts[0] = 0
    scale = 1.13 / hd ** 0.5
    args = (to_np(q), to_np(k), to_np(v), to_np(pos), to_np(starts), scale)
    kw = dict(k_scale=None if ks is None else to_np(ks), v_scale=None if vs is None else to_np(vs))
    out = decode_attn.decode_attention_ref(*args, **kw)
    np.testing.assert_allclose(out, _sdpa(q, k, v, ks, vs, pos, starts, scale, 0, False), atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(out, decode_attn.decode_attention_rows(*args, **kw), atol=2e-5, rtol=2e-5)
    if int8:
        c = cbind.decode_attn_i8(to_np(q), to_np(k), to_np(v), to_np(ks), to_np(vs), to_np(pos), to_np(starts), scale)
        np.testing.assert_allclose(c, out, atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("W,hd,G", [(128, 128, 5), (256, 64, 8), (100, 128, 4), (8, 16, 2)])
def test_ring_edge_vectors(W, hd, G):
    """tests/test_math_kernels.py:55-70: positions before, at and past the wrap; left pad past the window start."""
    B = 12
    q, k, v, ks, vs = attn_case(B, 1, G, hd, W, True, seed=1)
    pos = torch.tensor([0, 5, W - 2, W - 1, W, W + 1, 2 * W + 7, 3 * W - 1, 5 * W + 3, W + 10, 4 * W, 7])
    starts = torch.tensor([0, 2, 0, 3, 0, 4, 0, 2 * W + 5, 0, 30, 4 * W - 3, 7])
    starts = torch.minimum(starts, pos)
    args = (to_np(q), to_np(k), to_np(v), to_np(pos), to_np(starts), 0.1)
    kw = dict(window=W, k_scale=to_np(ks), v_scale=to_np(vs))
    out = decode_attn.decode_attention_ref(*args, **kw)
    np.testing.assert_allclose(out, _sdpa(q, k, v, ks, vs, pos, starts, 0.1, W, True), atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(out, decode_attn.decode_attention_rows(*args, **kw), atol=2e-5, rtol=2e-5)
    c = cbind.decode_attn_i8(to_np(q), to_np(k), to_np(v), to_np(ks), to_np(vs), to_np(pos), to_np(starts), 0.1, window=W)
    np.testing.assert_allclose(c, out, atol=2e-5, rtol=2e-5)


def test_window_on_linear_cache():
    """tests/test_math_kernels.py:73-82."""
    B, S, W = 6, 500, 64
    q, k, v, _, _ = attn_case(B, 1, 4, 128, S, False, seed=2)
    pos = torch.tensor([10, 63, 64, 200, 499, 300])
    starts = torch.tensor([0, 0, 1, 180, 0, 290])
    out = decode_attn.decode_attention_ref(to_np(q), to_np(k), to_np(v), to_np(pos), to_np(starts), 0.1, window=W, ring=False)
    np.testing.assert_allclose(out, _sdpa(q, k, v, None, None, pos, starts, 0.1, W, False), atol=2e-5, rtol=2e-5)
    lo, p = decode_attn.key_range(to_np(pos), to_np(starts), W)
    assert list(lo) == [0, 0, 1, 180, 436, 290] and list(p - lo + 1) == [11, 64, 64, 21, 64, 11]


def test_single_key_and_algorithmic_bytes():
    q, k, v, ks, vs = attn_case(2, 1, 8, 64, 32, True, seed=3)
    pos, starts = np.array([0, 9]), np.array([0, 9])
    out = decode_attn.decode_attention_ref(to_np(q), to_np(k), to_np(v), pos, starts, 0.14125, k_scale=to_np(ks), v_scale=to_np(vs))
    for b in range(2):  # one key: output is that key's dequantized value for every head
        exp = to_np(v)[b, 0, pos[b]].astype(np.float32) * np.float32(to_np(vs)[b, 0, pos[b]])
        np.testing.assert_allclose(out[b], np.broadcast_to(exp, (8, 64)), rtol=1e-6)
    assert decode_attn.algorithmic_bytes(pos, starts, 0, 2, 8, 1, 64) == 132 * 2 + 4 * 2 * 8 * 64 + 32


@pytest.mark.parametrize("window", [None, 256])
def test_varlen_matches_sdpa_per_segment(window):
    """tests/test_perf_opt.py:40-61: lens [300, 1000, 57, 700, 1], (N, 8, 64) / (N, 1, 64)."""
    lens = [300, 1000, 57, 700, 1]
    N = sum(lens)
    g = torch.Generator().manual_seed(0)
    q, k, v = torch.randn(N, 8, 64, generator=g), torch.randn(N, 1, 64, generator=g), torch.randn(N, 1, 64, generator=g)
    cu = np.concatenate([[0], np.cumsum(lens)])
    out = varlen_attn.varlen_attention_ref(q.numpy(), k.numpy(), v.numpy(), cu, 0.14125, window)
    for a, b in zip(cu[:-1], cu[1:]):
        Lq = b - a
        i = torch.arange(Lq)
        d = i[:, None] - i[None, :]
        m = d >= 0
        if window:
            m &= d < window
        z = torch.nn.functional.scaled_dot_product_attention(q[a:b].double().transpose(0, 1), k[a:b].double().transpose(0, 1).expand(8, Lq, 64),
                                                             v[a:b].double().transpose(0, 1).expand(8, Lq, 64), attn_mask=m, scale=0.14125)
        np.testing.assert_allclose(out[a:b], z.transpose(0, 1).numpy(), atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("window", [None, 3])
def test_varlen_grad_matches_finite_differences_and_autograd(window):
    """Pins oracle.varlen_attn.varlen_attention_grad_ref twice: by central differences of the forward restatement (float64,
    every input element of a tiny ragged case with an empty segment and grouped kv heads), and by torch autograd through a
    masked softmax written with torch ops (the formulation of the reference's test, tests/test_perf_opt.py:40-61)."""
    rng = np.random.default_rng(7)
    lens = [4, 0, 6, 1]
    N, H, K, hd, sc = sum(lens), 4, 2, 8, 0.37
    cu = np.concatenate([[0], np.cumsum(lens)])
    q, k, v, go = (rng.standard_normal(s_) for s_ in ((N, H, hd), (N, K, hd), (N, K, hd), (N, H, hd)))

    def fwd64(q_, k_, v_):   # the forward restatement, in float64
        out = np.zeros((N, H, hd))
        for a, b in zip(cu[:-1], cu[1:]):
            if b == a:
                continue
            i = np.arange(b - a)
            d = i[:, None] - i[None, :]
            m = (d >= 0) & ((d < window) if window else True)
            for h in range(H):
                s_ = np.where(m, q_[a:b, h] @ k_[a:b, h // (H // K)].T * sc, -np.inf)
                w = np.exp(s_ - s_.max(-1, keepdims=True))
                out[a:b, h] = (w / w.sum(-1, keepdims=True)) @ v_[a:b, h // (H // K)]
        return out
    np.testing.assert_allclose(fwd64(q, k, v), varlen_attn.varlen_attention_ref(q, k, v, cu, sc, window), atol=2e-6)
    dq, dk, dv = varlen_attn.varlen_attention_grad_ref(q, k, v, go, cu, sc, window)
    eps = 1e-6
    for x, gx, idx in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        num = np.zeros_like(x)
        for pos in np.ndindex(x.shape):
            args = [q.copy(), k.copy(), v.copy()]
            args[idx][pos] += eps
            up = (fwd64(*args) * go).sum()
            args[idx][pos] -= 2 * eps
            num[pos] = (up - (fwd64(*args) * go).sum()) / (2 * eps)
        np.testing.assert_allclose(gx, num, atol=2e-8 + 1e-6 * np.abs(num).max())
    # torch autograd
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    outs = []
    for a, b in zip(cu[:-1], cu[1:]):
        if b == a:
            continue
        i = torch.arange(b - a)
        d = i[:, None] - i[None, :]
        m = (d >= 0) & ((d < window) if window else torch.ones_like(d, dtype=torch.bool))
        kk = tk[a:b].repeat_interleave(H // K, dim=1).transpose(0, 1)
        vv = tv[a:b].repeat_interleave(H // K, dim=1).transpose(0, 1)
        s_ = (tq[a:b].transpose(0, 1) @ kk.transpose(1, 2) * sc).masked_fill(~m, float("-inf"))
        outs.append((s_.softmax(-1) @ vv).transpose(0, 1))
    (torch.cat(outs) * torch.tensor(go)).sum().backward()
    for gx, t in ((dq, tq), (dk, tk), (dv, tv)):
        np.testing.assert_allclose(gx, t.grad.numpy(), atol=1e-12, rtol=1e-10)
