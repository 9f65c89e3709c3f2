"""GPU parity: HIP kernels (through the C ABI, via the ultraviolet_amd.kernels mirror) vs the CPU oracle.

The cases restate the reference's kernel tests (tests/test_math_kernels.py, tests/test_perf_fz.py) on the same shapes
and edge vectors.  Bars: int8 bytes / fp16 scales / indices bit-exact; attention atol = rtol = 2e-3 on the rounded
output (the reference's own criterion, test_math_kernels.py:52) and 2e-3 relative on the fp32 pre-rounding output."""
import numpy as np
import pytest
import torch

from util import attn_case, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _oracle():
    from oracle import decode_attn, fused_sample, kv_quant, philox
    return decode_attn, fused_sample, kv_quant, philox


def _attn_check(q, k, v, ks, vs, pos, starts, scale, window=0, ring=None, splits=None, kview=None):
    """Run kernel (fp32 output and rounded output) and compare with the oracle."""
    from ultraviolet_amd.kernels import decode_attention
    da = _oracle()[0]
    d = lambda t: None if t is None else t.to(DEV)
    kk, vv, kss, vss = (d(k), d(v), d(ks), d(vs))
    if kview is not None:
        kk, vv = kk[:, :, :kview], vv[:, :, :kview]
        if kss is not None:
            kss, vss = kss[:, :, :kview], vss[:, :, :kview]
    kw = dict(window=window, ring=ring, k_scale=kss, v_scale=vss, num_splits=splits)
    out32 = decode_attention(d(q), kk, vv, d(pos), d(starts), scale, out_fp32=True, **kw)
    out = decode_attention(d(q), kk, vv, d(pos), d(starts), scale, **kw)
    torch.cuda.synchronize()
    ref = da.decode_attention_ref(to_np(q), to_np(k), to_np(v), to_np(pos), to_np(starts), scale, window=window,
                                  ring=ring, k_scale=None if ks is None else to_np(ks),
                                  v_scale=None if vs is None else to_np(vs))
    o32 = to_np(out32)
    assert np.isfinite(o32).all()
    np.testing.assert_allclose(o32, ref, atol=2e-3, rtol=2e-3)
    np.testing.assert_allclose(to_np(out), ref.astype(np.float32), atol=2e-3 + 4e-3 * np.abs(ref).max() * (q.dtype == torch.bfloat16),
                               rtol=2e-3 if q.dtype == torch.float16 else 8e-3)
    return o32, ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("int8", [False, True])
@pytest.mark.parametrize("B,KH,G,hd", [(1, 1, 1, 128), (3, 1, 4, 128), (17, 1, 5, 128), (5, 2, 4, 64),
                                       (9, 1, 8, 64), (4, 2, 2, 16), (6, 1, 7, 128), (33, 1, 8, 64)])
@pytest.mark.parametrize("splits", [1, 3, None])
def test_global_ragged(dtype, int8, B, KH, G, hd, splits):
    """reference: tests/test_math_kernels.py:36-52."""
    S = 700
    q, k, v, ks, vs = attn_case(B, KH, G, hd, S, int8, dtype=dtype)
    g = torch.Generator().manual_seed(1)
    pos = torch.randint(0, S, (B,), generator=g)
    pos[0] = S - 1
    starts = (torch.rand(B, generator=g) * (pos + 1).float()).long()
    starts[0] = 0
    _attn_check(q, k, v, ks, vs, pos, starts, 1.13 / hd ** 0.5, splits=splits)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,S,ring", [(3, 1056, False), (200, 1056, False), (300, 2080, False), (500, 1024, False), (40, 1024, True)])
def test_few_and_many_rows_on_long_caches(dtype, B, S, ring):
    """Caches of >= 1024 slots with 3 .. 500 rows: rows from one key to the whole cache, left-padded starts, a ring of 1024
    slots several times around - rows that leave most of a workgroup's waves without a tile next to rows that fill it."""
    q, k, v, ks, vs = attn_case(B, 1, 8, 64, S, True, dtype=dtype)
    g = torch.Generator().manual_seed(B + S)
    pos = torch.randint(0, S if not ring else 5 * S, (B,), generator=g)
    pos[0], pos[1 % B] = (S - 1 if not ring else 3 * S + 17), 0
    starts = (torch.rand(B, generator=g) * (pos + 1).float()).long()
    starts[0] = 0
    _attn_check(q, k, v, ks, vs, pos, starts, 1.13 / 8, window=S if ring else 0, ring=ring)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,S,ring,G", [(3, 1056, False, 8), (200, 1056, False, 8), (300, 2080, False, 4), (40, 1024, True, 8), (64, 256, True, 2),
                                        (50, 100, False, 8)])
def test_unquantized_cache_on_the_mfma_kernel(dtype, B, S, ring, G):
    """K / V cached unquantized in the q dtype (the reference's accuracy baseline, fast_decode.py:21-57 with kv_dtype fp16):
    head_dim 64 runs on the MFMA kernel too - 1, 2 and 4 waves per row, ring wrap-around, left-padded starts, a cache that
    ends inside a super-tile - and slots outside lo..pos may hold NaN patterns."""
    from ultraviolet_amd.kernels import decode_attention
    from ultraviolet_amd.kernels.decode_attn import supported
    q, k, v, _, _ = attn_case(B, 1, G, 64, S, False, dtype=dtype, seed=B)
    g = torch.Generator().manual_seed(B + S)
    pos = torch.randint(0, S if not ring else 5 * S, (B,), generator=g)
    pos[0], pos[1 % B] = (S - 1 if not ring else 3 * S + 17), 0
    starts = (torch.rand(B, generator=g) * (pos + 1).float()).long()
    starts[0] = 0
    d = lambda t: t.to(DEV)
    assert supported(d(q), d(k))
    o32, ref = _attn_check(q, k, v, None, None, pos, starts, 1.13 / 8, window=S if ring else 0, ring=ring)
    if not ring:   # poison what no row may read
        k2, v2 = k.clone(), v.clone()
        for b in range(B):
            bad = torch.ones(S, dtype=torch.bool)
            bad[starts[b]:pos[b] + 1] = False
            k2[b, 0, bad] = float("nan")
            v2[b, 0, bad] = float("nan")
        out = decode_attention(d(q), d(k2), d(v2), d(pos), d(starts), 1.13 / 8, out_fp32=True)
        assert torch.equal(out.cpu(), torch.from_numpy(o32))


@pytest.mark.parametrize("int8", [False, True])
@pytest.mark.parametrize("W,hd,G", [(128, 128, 5), (256, 64, 8), (1024, 128, 4), (100, 128, 4), (64, 64, 8),
                                    (100, 64, 8)])
@pytest.mark.parametrize("splits", [1, 4])
def test_ring_wraparound(int8, W, hd, G, splits):
    """reference: tests/test_math_kernels.py:55-70 (positions before, at and past the wrap; left pad past window start)."""
    B = 12
    q, k, v, ks, vs = attn_case(B, 1, G, hd, W, int8, seed=1)
    pos = torch.tensor([0, 5, W - 2, W - 1, W, W + 1, 2 * W + 7, 3 * W - 1, 5 * W + 3, W + 10, 4 * W, 7])
    starts = torch.tensor([0, 2, 0, 3, 0, 4, 0, 2 * W + 5, 0, 30, 4 * W - 3, 7])
    _attn_check(q, k, v, ks, vs, pos, starts, 0.1, window=W, splits=splits)


@pytest.mark.parametrize("int8,hd,G", [(False, 128, 4), (True, 64, 8)])
def test_window_smaller_than_cache(int8, hd, G):
    """Sliding window on a non-ring cache; reference: tests/test_math_kernels.py:73-82."""
    B, S, W = 6, 500, 64
    q, k, v, ks, vs = attn_case(B, 1, G, hd, S, int8, seed=2)
    pos = torch.tensor([10, 63, 64, 200, 499, 300])
    starts = torch.tensor([0, 0, 1, 180, 0, 290])
    _attn_check(q, k, v, ks, vs, pos, starts, 0.1, window=W, ring=False, splits=2)


def test_matches_sdpa_fp16():
    """Kernel vs torch SDPA with an additive mask (the model's formulation); reference: test_math_kernels.py:85-98."""
    from ultraviolet_amd.kernels import decode_attention
    B, G, hd, S = 32, 5, 128, 2048
    q, k, v, _, _ = attn_case(B, 1, G, hd, S, False, seed=3)
    g = torch.Generator().manual_seed(3)
    pos = torch.randint(S // 2, S, (B,), generator=g)
    starts = torch.randint(0, 50, (B,), generator=g)
    t = torch.arange(S)[None]
    bias = torch.zeros(B, S).masked_fill(~((t <= pos[:, None]) & (t >= starts[:, None])), float("-inf"))
    bias = bias[:, None, None].expand(B, 1, G, S)
    z = torch.nn.functional.scaled_dot_product_attention(q.float().view(B, 1, G, hd), k.float(), v.float(),
                                                         attn_mask=bias, scale=0.1)
    out = decode_attention(q.to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), starts.to(DEV), 0.1)
    torch.testing.assert_close(out.float().cpu().view_as(z), z, atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("hd,G,KH", [(128, 4, 2), (64, 8, 1), (64, 4, 2)])
def test_non_contiguous_global_slice(hd, G, KH):
    """cache[:, :, :g_len] views: strides must be honoured; reference: tests/test_math_kernels.py:101-112."""
    B, S = 5, 512
    q, k, v, ks, vs = attn_case(B, KH, G, hd, S, True, seed=4)
    pos = torch.tensor([0, 100, 255, 17, 200])
    starts = torch.tensor([0, 3, 0, 17, 150])
    _attn_check(q, k, v, ks, vs, pos, starts, 0.1, splits=2, kview=256)


def test_int32_positions_and_empty_rows():
    from ultraviolet_amd.kernels import decode_attention
    B, S = 7, 256
    q, k, v, ks, vs = attn_case(B, 1, 8, 64, S, True, seed=5, dtype=torch.bfloat16)
    pos = torch.tensor([0, 1, 31, 32, 33, 255, 128], dtype=torch.int32)
    starts = torch.tensor([0, 1, 0, 32, 0, 200, 129], dtype=torch.int32)  # last row: start > pos -> no valid key
    d = lambda t: t.to(DEV)
    out = decode_attention(d(q), d(k), d(v), d(pos), d(starts), 0.14125, k_scale=d(ks), v_scale=d(vs), num_splits=2,
                           out_fp32=True)
    da = _oracle()[0]
    ref = da.decode_attention_ref(to_np(q)[:6], to_np(k)[:6], to_np(v)[:6], to_np(pos)[:6], to_np(starts)[:6], 0.14125,
                                  k_scale=to_np(ks)[:6], v_scale=to_np(vs)[:6])
    o = to_np(out)
    np.testing.assert_allclose(o[:6], ref, atol=2e-3, rtol=2e-3)
    assert (o[6] == 0).all()


def test_stale_nonfinite_scales_outside_range_are_ignored():
    """Slots outside lo..pos may hold anything (caches are never cleared on refill: reference model.py:883-884)."""
    from ultraviolet_amd.kernels import decode_attention
    B, S = 4, 128
    q, k, v, ks, vs = attn_case(B, 1, 8, 64, S, True, seed=6)
    pos = torch.tensor([40, 77, 5, 100])
    starts = torch.tensor([3, 70, 0, 64])
    ks2, vs2 = ks.clone(), vs.clone()
    for b in range(B):
        bad = torch.ones(S, dtype=torch.bool)
        bad[starts[b]:pos[b] + 1] = False
        ks2[b, 0, bad] = float("nan")
        vs2[b, 0, bad] = float("inf")
    d = lambda t: t.to(DEV)
    for sp in (1, 3):
        out = decode_attention(d(q), d(k), d(v), d(pos), d(starts), 0.1, k_scale=d(ks2), v_scale=d(vs2), num_splits=sp,
                               out_fp32=True)
        ref = _oracle()[0].decode_attention_ref(to_np(q), to_np(k), to_np(v), to_np(pos), to_np(starts), 0.1,
                                                k_scale=to_np(ks), v_scale=to_np(vs))
        np.testing.assert_allclose(to_np(out), ref, atol=2e-3, rtol=2e-3)


def test_config2_shape_relative_error():
    """BASELINE config 2: 256 rows, 8 heads x 64, KH = 1, contexts U[64, 1024], bf16 q, int8 KV, scale 0.14125.
    Bar: 2e-3 max relative error on the fp32-accumulation output, relative error of a (row, head) output vector being
    max_d |out - ref| / max_d |ref|; plus the reference's elementwise atol = rtol = 2e-3."""
    from ultraviolet_amd.kernels import decode_attention
    B, S = 256, 1024
    q, k, v, ks, vs = attn_case(B, 1, 8, 64, S, True, seed=0, dtype=torch.bfloat16)
    rng = np.random.default_rng(0)
    n = rng.integers(64, 1025, size=B)
    pos = torch.from_numpy(n - 1)
    starts = torch.zeros(B, dtype=torch.long)
    d = lambda t: t.to(DEV)
    ref = _oracle()[0].decode_attention_ref(to_np(q), to_np(k), to_np(v), to_np(pos), to_np(starts), 0.14125,
                                            k_scale=to_np(ks), v_scale=to_np(vs))
    for sp in (1, 2, None):
        out = to_np(decode_attention(d(q), d(k), d(v), d(pos), d(starts), 0.14125, k_scale=d(ks), v_scale=d(vs),
                                     num_splits=sp, out_fp32=True))
        rel = np.abs(out - ref).max(-1) / np.abs(ref).max(-1)
        assert rel.max() < 2e-3, rel.max()
        np.testing.assert_allclose(out, ref, atol=2e-3, rtol=2e-3)


# ------------------------------------------------------------------------------------------------ quantizer
def _all_patterns(dtype):
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(dtype)
    return x[torch.isfinite(x.float())]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hd", [64, 128, 16, 48])
def test_quantize_bit_exact_all_patterns(dtype, hd):
    """Every finite fp16 / bf16 bit pattern appears as an element, against rows whose absmax sweeps every pattern."""
    from ultraviolet_amd.kernels import quantize_kv
    kq = _oracle()[2]
    vals = _all_patterns(dtype)
    g = torch.Generator().manual_seed(hd)
    n = vals.numel()
    rows = (n + hd - 1) // hd * 4
    idx = torch.randint(0, n, (rows, hd), generator=g)
    idx.view(-1)[:n] = torch.arange(n)
    x = vals[idx]
    # scale rows so the absmax also sweeps magnitudes: keep some rows as is, shrink others
    mags = vals[torch.randint(0, n, (rows, 1), generator=g)].float().abs().clamp(max=6e4)
    x2 = torch.where(x.float().abs() <= mags, x, torch.zeros_like(x))
    x = torch.cat([x, x2])
    q, s = quantize_kv(x.to(DEV))
    rq, rs = kq.quantize_kv(to_np(x))
    assert np.array_equal(to_np(q), rq)
    assert np.array_equal(to_np(s).view(np.uint16), rs.view(np.uint16))


def test_quantize_fp32_rows_and_zero_row():
    from ultraviolet_amd.kernels import dequantize_kv, quantize_kv
    kq = _oracle()[2]
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 3, 128, generator=g) * 3
    x[0, 0] = 0
    x[1, 1] = 1e-9       # scale underflows fp16 -> s = 0, codes +-127
    x[2, 2, 5] = 7e4     # absmax/127 fine
    q, s = quantize_kv(x.to(DEV))
    rq, rs = kq.quantize_kv(x.numpy())
    assert np.array_equal(to_np(q), rq) and np.array_equal(to_np(s).view(np.uint16), rs.view(np.uint16))
    assert (to_np(q)[0, 0] == 0).all()
    # reference bound, tests/test_math_kernels.py:115-121
    xh = x.clamp(-100, 100).half()  # 7e4 is not finite in fp16
    q, s = quantize_kv(xh.to(DEV))
    err = (dequantize_kv(q, s).float().cpu() - xh.float()).abs()
    assert err.max() <= (s.float().cpu().unsqueeze(-1) * 0.5 + 1e-3).max()


def test_kv_write_flat_index():
    """reference: tests/test_math_kernels.py:122-128 (idx = [3, 31, 32, 55])."""
    from ultraviolet_amd.kernels import dequantize_kv, kv_write
    kq = _oracle()[2]
    g = torch.Generator().manual_seed(0)
    cache = torch.zeros(4, 1, 16, 128, dtype=torch.int8)
    sc = torch.zeros(4, 1, 16, dtype=torch.half)
    idx = torch.tensor([0 * 16 + 3, 1 * 16 + 15, 2 * 16 + 0, 3 * 16 + 7])
    xv = torch.randn(4, 128, generator=g).half()
    c_d, s_d = cache.to(DEV), sc.to(DEV)
    kv_write(c_d, s_d, idx.to(DEV), xv.to(DEV))
    rc, rs = cache.numpy().copy(), sc.numpy().copy()
    kq.kv_write(rc, rs, idx.numpy(), to_np(xv))
    assert np.array_equal(to_np(c_d), rc) and np.array_equal(to_np(s_d).view(np.uint16), rs.view(np.uint16))
    back = dequantize_kv(c_d.view(-1, 128)[idx.to(DEV)], s_d.view(-1)[idx.to(DEV)])
    torch.testing.assert_close(back.float().cpu(), xv.float(), atol=0.03, rtol=0.03)
    # unquantized cache
    c16 = torch.zeros(4, 1, 16, 128, dtype=torch.half, device=DEV)
    kv_write(c16, None, idx.to(DEV), xv.to(DEV))
    assert torch.equal(c16.view(-1, 128)[idx.to(DEV)].cpu(), xv)


@pytest.mark.parametrize("ring", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_kv_append_matches_oracle_writes(ring, dtype):
    """Fused K+V append == two oracle kv_write calls at (b*K+h)*S + pos (or pos % S)."""
    from ultraviolet_amd.kernels import kv_append
    kq = _oracle()[2]
    B, K, S, hd = 37, 2, 48, 64
    g = torch.Generator().manual_seed(3)
    kc = torch.randint(-127, 128, (B, K, S, hd), generator=g, dtype=torch.int8)
    vc = torch.randint(-127, 128, (B, K, S, hd), generator=g, dtype=torch.int8)
    ksc = torch.rand(B, K, S, generator=g).half()
    vsc = torch.rand(B, K, S, generator=g).half()
    k = torch.randn(B, K, hd, generator=g).to(dtype)
    v = torch.randn(B, K, hd, generator=g).to(dtype)
    pos = torch.randint(0, 5 * S if ring else S, (B,), generator=g)
    d = lambda t: t.to(DEV)
    kcd, vcd, ksd, vsd = d(kc), d(vc), d(ksc), d(vsc)
    kv_append(d(k), d(v), kcd, vcd, ksd, vsd, d(pos), ring=ring)
    rk, rv, rks, rvs = kc.numpy().copy(), vc.numpy().copy(), ksc.numpy().copy(), vsc.numpy().copy()
    ix = kq.decode_flat_index(pos.numpy(), K, S, ring)
    kq.kv_write(rk, rks, ix, to_np(k).reshape(-1, hd))
    kq.kv_write(rv, rvs, ix, to_np(v).reshape(-1, hd))
    assert np.array_equal(to_np(kcd), rk) and np.array_equal(to_np(vcd), rv)
    assert np.array_equal(to_np(ksd).view(np.uint16), rks.view(np.uint16))
    assert np.array_equal(to_np(vsd).view(np.uint16), rvs.view(np.uint16))


def test_kv_write_rows_prefill():
    """reference semantics of kv_write_rows (kv_quant.py:39-54): partial rows, ring slots."""
    from ultraviolet_amd.kernels import kv_write_rows
    kq = _oracle()[2]
    B, K, S, hd, T = 6, 1, 16, 64, 21
    g = torch.Generator().manual_seed(4)
    cache = torch.randint(-5, 5, (B, K, S, hd), generator=g, dtype=torch.int8)
    sc = torch.rand(B, K, S, generator=g).half()
    new = torch.randn(3, K, T, hd, generator=g).half()
    rows = torch.tensor([4, 0, 3])
    lo = T - S
    slots = torch.arange(lo, T) % S
    cd, sd = cache.to(DEV), sc.to(DEV)
    kv_write_rows(cd, sd, new[:, :, lo:].to(DEV), slots.to(DEV), rows.to(DEV))
    rc, rs = cache.numpy().copy(), sc.numpy().copy()
    kq.kv_write_rows(rc, rs, to_np(new[:, :, lo:]), slots.numpy(), rows.numpy())
    assert np.array_equal(to_np(cd), rc) and np.array_equal(to_np(sd).view(np.uint16), rs.view(np.uint16))


# ------------------------------------------------------------------------------------------------ sampler
SC = (23.0, 5.0, 7.5)


@pytest.mark.parametrize("T", [1.0, 0.8])
@pytest.mark.parametrize("dtype,V", [(torch.float16, 16384), (torch.bfloat16, 32768)])
def test_sampler_matches_ref(T, dtype, V):
    """reference: tests/test_perf_fz.py:96-119: token is the inverse-CDF draw of the exact (fp64) softmax up to fp32
    summation rounding; mostly the same token as the flat-cumsum oracle; log-probs match log_softmax."""
    from ultraviolet_amd.kernels.fused_sample import fused_sample
    fs = _oracle()[1]
    g = torch.Generator().manual_seed(0)
    B = 1024
    x = (torch.randn(B, V, generator=g) * torch.rand(B, 1, generator=g) * 8).to(dtype)
    u = torch.rand(B, generator=g)
    t, lp = fused_sample(x.to(DEV), u.to(DEV), SC, T)
    t, lp = t.cpu(), lp.cpu()
    tr, lpr = fs.fused_sample_ref(to_np(x), u.numpy(), SC, T)
    assert t.dtype == torch.int64 and t.min() >= 0 and t.max() < V
    # The oracle's flat sequential fp32 cumsum and the kernel's chunk / lane / element sums are different summation
    # orders of the same masses, so tokens agree only up to fp32 summation error (which grows with V for the flat
    # sum); the order-independent checks are agreement with the float64 inverse-CDF draw and its CDF interval.
    assert (t.numpy() == tr).mean() > 0.9
    z = torch.from_numpy(fs.softcap(to_np(x), SC)).double()
    e = torch.exp((z - SC[0]) / T)
    cs = e.cumsum(-1)
    S = cs[:, -1]
    tgt = (1.0 - u.double()) * S
    hi = cs.gather(1, t[:, None])[:, 0]
    lo = hi - e.gather(1, t[:, None])[:, 0]
    tol = 1e-5 * S
    assert ((tgt >= lo - tol) & (tgt <= hi + tol)).all()
    t64 = torch.searchsorted(cs, tgt[:, None]).squeeze(1).clamp_(max=V - 1)
    assert (t == t64).float().mean() > 0.99
    ls = torch.log_softmax(z / T, -1).gather(1, t[:, None])[:, 0]
    assert (lp.double() - ls).abs().max() < 2e-5


def test_sampler_edges():
    """reference: tests/test_perf_fz.py:66-71."""
    from ultraviolet_amd.kernels.fused_sample import fused_sample
    x = torch.full((2, 512), -1e4)
    x[:, 40] = 10.0
    tok, lp = fused_sample(x.to(DEV), torch.tensor([0.0, 1.0 - 2 ** -24]).to(DEV), SC, 1.0)
    assert tok.max() < 512 and tok.min() >= 0 and torch.isfinite(lp).all()


def test_sampler_distribution_chi2():
    """reference: tests/test_perf_fz.py:122-134."""
    from ultraviolet_amd.kernels.fused_sample import fused_sample
    fs = _oracle()[1]
    g = torch.Generator().manual_seed(1)
    V, n = 4096, 1 << 17
    for scale in (2.0, 12.0):
        x = (torch.randn(V, generator=g) * scale).half()
        p = torch.softmax(torch.from_numpy(fs.softcap(to_np(x), SC)).double(), -1)
        u = torch.rand(n, generator=g)
        t, _ = fused_sample(x[None].expand(n, V).contiguous().to(DEV), u.to(DEV), SC, 1.0)
        cnt = torch.bincount(t.cpu(), minlength=V).double()
        e = p * n
        big = e >= 5
        obs = torch.cat([cnt[big], cnt[~big].sum()[None]])
        ex = torch.cat([e[big], e[~big].sum()[None]])
        chi = ((obs - ex) ** 2 / ex).sum()
        df = int(big.sum())
        pval = float(torch.special.gammaincc(torch.tensor(df / 2, dtype=torch.float64), chi / 2))
        assert pval > 1e-3


def test_sampler_seeded_philox_and_greedy():
    from ultraviolet_amd.kernels.fused_sample import fused_sample, fused_sample_seeded, greedy_sample
    _, fs, _, ph = _oracle()
    g = torch.Generator().manual_seed(2)
    B, V = 300, 2048
    x = (torch.randn(B, V, generator=g) * 4).bfloat16()
    req = torch.randint(0, 2 ** 40, (B,), generator=g)
    ti = torch.randint(0, 4096, (B,), generator=g)
    seed = 0x1234_5678_9ABC_DEF0
    t1, lp1, u1 = fused_sample_seeded(x.to(DEV), seed, req.to(DEV), ti.to(DEV), SC, 1.0, return_u=True)
    uref = ph.request_uniform(seed, req.numpy(), ti.numpy())
    assert np.array_equal(u1.cpu().numpy(), uref)            # Philox stream is bit-exact
    t2, lp2 = fused_sample(x.to(DEV), torch.from_numpy(uref).to(DEV), SC, 1.0)
    assert torch.equal(t1, t2) and torch.equal(lp1, lp2)
    tg, lpg = greedy_sample(x.to(DEV), SC)
    z = fs.softcap(to_np(x), SC)
    assert np.array_equal(tg.cpu().numpy(), np.argmax(to_np(x), -1))
    ref = torch.log_softmax(torch.from_numpy(z).double(), -1).gather(1, tg.cpu()[:, None])[:, 0]
    assert (lpg.cpu().double() - ref).abs().max() < 2e-5


def test_error_paths_are_loud():
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels import decode_attention, quantize_kv
    with pytest.raises(L.UvmiError):
        quantize_kv(torch.zeros(4, 64))  # CPU tensor: no fallback
    q = torch.zeros(2, 8, 64, device=DEV, dtype=torch.float64)  # queries are fp16, bf16 or fp32
    kc = torch.zeros(2, 1, 64, 64, dtype=torch.int8, device=DEV)
    sc = torch.zeros(2, 1, 64, dtype=torch.half, device=DEV)
    p = torch.zeros(2, dtype=torch.long, device=DEV)
    with pytest.raises((L.UvmiError, KeyError)):
        decode_attention(q, kc, kc, p, p, 0.1, k_scale=sc, v_scale=sc)
    with pytest.raises((L.UvmiError, AssertionError)):
        decode_attention(q.half(), kc, kc, p, p, 0.1)          # an int8 cache without its scales


def test_fp32_queries_stay_fp32():
    """q in fp32 takes the plain fp32 kernel - no 16-bit rounding of q or of the probabilities: against the float64 oracle
    it is two orders of magnitude closer than the 2e-3 bar of the 16-bit paths (int8 and fp32 caches, ring and linear)."""
    from oracle import decode_attn as odec
    from ultraviolet_amd.kernels import decode_attention
    from util import attn_case
    for ring in (False, True):
        q, k, v, ks, vs = attn_case(7, 1, 8, 64, 128, True, seed=21 + ring, dtype=torch.float32)
        pos = torch.tensor([0, 5, 127, 200, 64, 31, 129]) if ring else torch.tensor([0, 5, 127, 90, 64, 31, 100])
        starts = torch.tensor([0, 2, 0, 120, 0, 30, 60]) if ring else torch.tensor([0, 2, 0, 50, 0, 30, 60])
        w = 128 if ring else 0
        out = decode_attention(q.to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), starts.to(DEV), 0.14125, window=w, ring=ring,
                               k_scale=ks.to(DEV), v_scale=vs.to(DEV))
        assert out.dtype == torch.float32
        ref = odec.decode_attention_ref(q.double().numpy(), k.numpy(), v.numpy(), pos.numpy(), starts.numpy(), 0.14125, window=w, ring=ring,
                                        k_scale=ks.numpy(), v_scale=vs.numpy())
        np.testing.assert_allclose(out.cpu().numpy(), ref, atol=2e-5, rtol=2e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rope_table_matches_rounded_cos_sin(dtype):
    """uvmi_rope_table: row p = cos(p * inv_freq) then sin(p * inv_freq), each rounded to the activation type - compared with
    float64 cos / sin of the fp32 angle (the reference's Rotary buffers, ultraviolet/model.py:198-226): at most one unit
    in the last place of the rounding type apart (fp32 cosf against float64), and exactly representable in that type."""
    from ultraviolet_amd.kernels.decode_attn import rope_table
    inv = ((1.0 / 1024.0) ** torch.linspace(0, 1, 16, dtype=torch.float32)).cuda()
    n = 2336
    tab = rope_table(inv, n, dtype)
    assert tab.shape == (n, 32) and tab.dtype == torch.float32
    assert torch.equal(tab.to(dtype).float(), tab)
    ang = (torch.arange(n, dtype=torch.float32, device="cuda")[:, None] * inv[None, :]).double()
    ref = torch.cat([ang.cos(), ang.sin()], 1)
    ulp = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -23}[dtype]
    assert float((tab.double() - ref).abs().max()) <= ulp
    exact = ref.float().to(dtype).float()
    if dtype != torch.float32:   # (fp32 cosf itself is a unit off float64 now and then; a 16-bit rounding hides that
        assert float((tab != exact).float().mean()) < 1e-3   # except where the fp32 value lands across a rounding tie)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N", [(1, 640, 656), (64, 640, 656), (100, 512, 640), (128, 640, 3328), (257, 1664, 640), (384, 640, 48),
                                   (65, 64, 16), (200, 960, 96), (77, 1984, 32), (700, 640, 656), (1030, 2048, 208)])
def test_skinny_gemm_matches_fp32_reference(dtype, M, K, N):
    """uvmi_gemm_tn against a float64 product of the same 16-bit inputs: the result is the fp32-accumulated product rounded
    once to the activation type (tolerance: half a unit in the last place of the largest magnitude plus the accumulation
    error of K terms), on ragged M (rows past M cut off), N that is not a multiple of the strip, both strip widths (K
    below / above 960) and padded row pitches."""
    from ultraviolet_amd.kernels.gemm import gemm_tn, gemm_supported
    g = torch.Generator(device="cuda").manual_seed(M * 7 + N)
    a_full = torch.randn(M, K + 8, device="cuda", generator=g).to(dtype)
    w_full = (torch.randn(N, K + 16, device="cuda", generator=g) / K ** 0.5).to(dtype)
    a, w = a_full[:, :K], w_full[:, :K]
    assert gemm_supported(a, w)
    ref = a.double() @ w.double().t()
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    tol = ulp * ref.abs().clamp_min(1.0) + 1e-5 * K ** 0.5
    # 64-row workgroups; 16-row workgroups whose waves split K (the latter when K % 128 == 0); the tiled kernel with 128 x 128
    # and 64 x 64 tiles (any K); the library's own choice
    for config in ((1, 2) if K <= 1984 else ()) + (3, 4, 0):
        out_full = torch.full((M, N + 4), 7.0, device="cuda", dtype=dtype)
        out = out_full[:, :N]
        gemm_tn(a, w, out, config=config)
        assert bool(((out.double() - ref).abs() <= tol).all()), (config, float((out.double() - ref).abs().max()))
        assert bool((out_full[:, N:] == 7.0).all())   # nothing written past column N


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,f", [(3, 640, 1664), (128, 640, 1664), (200, 128, 48), (600, 640, 1664)])
def test_skinny_gemm_swiglu_epilogue(dtype, M, K, f):
    """The SWIGLU epilogue on interleaved gate / up rows equals the two-pass path (GEMM to the activation type, then
    silu(g) rounded, times u - ultraviolet/model.py:388-391) up to the GEMMs' own last-place differences."""
    from ultraviolet_amd.kernels.gemm import SWIGLU, gemm_tn, interleave_gate_up
    g = torch.Generator(device="cuda").manual_seed(M + f)
    a = torch.randn(M, K, device="cuda", generator=g).to(dtype)
    wg = (torch.randn(f, K, device="cuda", generator=g) / K ** 0.5).to(dtype)
    wu = (torch.randn(f, K, device="cuda", generator=g) / K ** 0.5).to(dtype)
    gg = (a.double() @ wg.double().t()).to(dtype).double()
    uu = (a.double() @ wu.double().t()).to(dtype).double()
    ref = (gg * torch.sigmoid(gg)).to(dtype).double() * uu
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    tol = 4 * ulp * ref.abs().clamp_min(1.0) + 4 * ulp * (gg.abs() + uu.abs())   # g and u may each sit one rounding step off
    for config in (1, 2, 3, 4):
        out = gemm_tn(a, interleave_gate_up(wg, wu), epilogue=SWIGLU, config=config)
        assert out.shape == (M, f)
        assert bool(((out.double() - ref).abs() <= tol).all()), (config, float((out.double() - ref).abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,f,d", [(1, 1664, 640), (300, 1664, 640), (37, 24, 10)])
def test_swiglu_with_folded_prenorm(dtype, rows, f, d):
    """uvmi_swiglu_norm(gu = h @ W.T, h) equals the SwiGLU of rmsnorm(h) @ W.T with the norm applied as a row scale of the
    product (ultraviolet/model.py:570, 388-391): restated here with torch in the same rounding order; the row scale may
    differ in its last fp32 place (summation order), which can move a rounded factor by one place of the activation type."""
    from ultraviolet_amd import _lib as L
    g = torch.Generator(device="cuda").manual_seed(rows + f)
    h = (3.0 * torch.randn(rows, d, device="cuda", generator=g)).to(dtype)
    gu = torch.randn(rows, 2 * f, device="cuda", generator=g).to(dtype)
    eps = 1e-6
    out = torch.full((rows + 1, f), 7.0, device="cuda", dtype=dtype)
    code = L.dtype_code(dtype)
    L.check(L.lib().uvmi_swiglu_norm(gu.data_ptr(), h.data_ptr(), code, rows, f, d, eps, out.data_ptr(), L.stream_ptr(gu)), "uvmi_swiglu_norm")
    rn = torch.rsqrt(h.float().pow(2).mean(-1, keepdim=True) + eps)
    gv, uv = (gu[:, :f].float() * rn).to(dtype).float(), (gu[:, f:].float() * rn).to(dtype).float()
    ref = ((gv * torch.sigmoid(gv)).to(dtype).float() * uv).to(dtype)
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    err = (out[:rows].float() - ref.float()).abs()
    assert bool((err <= 4 * ulp * ref.float().abs().clamp_min(0.05)).all()), float(err.max())
    assert float((out[:rows] != ref).float().mean()) < 0.02
    assert bool((out[rows] == 7.0).all())
    with pytest.raises(L.UvmiError):   # f must be a multiple of 8
        L.check(L.lib().uvmi_swiglu_norm(gu.data_ptr(), h.data_ptr(), code, rows, f + 1, d, eps, out.data_ptr(), L.stream_ptr(gu)), "uvmi_swiglu_norm")


@pytest.mark.gpu
def test_skinny_gemm_rejects_what_it_cannot_do():
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels.gemm import SWIGLU, gemm_supported, gemm_tn
    a = torch.zeros(4, 2048, device="cuda", dtype=torch.bfloat16)
    w = torch.zeros(32, 2048, device="cuda", dtype=torch.bfloat16)
    assert gemm_supported(a, w)                # K above 1984: the tiled kernel only
    gemm_tn(a, w)
    for config in (1, 2):
        with pytest.raises(L.UvmiError):
            gemm_tn(a, w, config=config)
    with pytest.raises(L.UvmiError):
        gemm_tn(a[:, :1000], w[:, :1000])      # K % 64 != 0
    with pytest.raises(L.UvmiError):
        gemm_tn(a[:, :1024], w[:, :1024], epilogue=SWIGLU, config=1)   # the skinny SwiGLU strip needs K <= 960
    gemm_tn(a[:, :1024], w[:, :1024], epilogue=SWIGLU)
    assert not gemm_supported(a.float(), w.float())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,V", [(torch.float32, 2048), (torch.bfloat16, 32768), (torch.float16, 16384)])
@pytest.mark.parametrize("T,top_k,top_p", [(1.0, 50, 1.0), (0.8, 0, 0.9), (1.0, 20, 0.5), (0.7, 1, 1.0), (1.0, 0, 0.05), (1.0, 5000, 0.999)])
def test_truncated_sampler_matches_oracle(dtype, V, T, top_k, top_p):
    """Top-k / nucleus sampling (sample(), ultraviolet/model.py:1194-1211) against the float64 oracle: the kept set (read
    back through the threshold output) is the oracle's except where a token's mass sits within rounding of the nucleus
    boundary; the token is a kept one, lies in the float64 CDF interval of the kept distribution for the row's uniform and
    is the oracle's own token almost always; log-probs are those of the untruncated softmax."""
    from ultraviolet_amd.kernels.fused_sample import sample_filtered
    fs = _oracle()[1]
    g = torch.Generator().manual_seed(V + top_k)
    B = 192
    x = (torch.randn(B, V, generator=g) * (torch.rand(B, 1, generator=g) * 6 + 0.5)).to(dtype)
    u = torch.rand(B, generator=g)
    t, lp, thr = sample_filtered(x.to(DEV), u.to(DEV), SC, T, top_k, top_p, return_threshold=True)
    t, lp, thr = t.cpu().numpy(), lp.cpu().double().numpy(), thr.cpu().double().numpy()
    xn = to_np(x).astype(np.float64)
    tr, lpr, keep = fs.sample_filtered_ref(xn, u.numpy(), SC, T, top_k, top_p)
    z = SC[0] / (1.0 + np.exp(-(xn + SC[1]) / SC[2]))
    e = np.exp((z - SC[0]) / T)
    kept_kernel = e >= thr[:, None] * (1 - 2e-6)
    same = (kept_kernel == keep).all(1)
    assert same.mean() >= 0.97, same.mean()
    for i in np.nonzero(~same)[0]:   # a differing row differs by the tie group at the cut only: its mass straddles top_p
        diff = kept_kernel[i] != keep[i]
        assert top_p < 1.0 and np.ptp(e[i][diff]) <= 1e-5 * e[i][diff].max()
    assert kept_kernel[np.arange(B), t].all()
    if top_k == 1:
        assert (t == xn.argmax(1)).all() or (z[np.arange(B), t] == z.max(1)).all()
    em = np.where(kept_kernel, e, 0.0)
    cs = em.cumsum(1)
    S = cs[:, -1]
    tgt = (1.0 - u.double().numpy()) * S
    hi = cs[np.arange(B), t]
    lo = hi - em[np.arange(B), t]
    assert ((tgt >= lo - 1e-5 * S) & (tgt <= hi + 1e-5 * S)).all()
    assert (t[same] == tr[same]).mean() > 0.98
    full = z / T - (z.max(1, keepdims=True) / T + np.log(np.exp((z - z.max(1, keepdims=True)) / T).sum(1, keepdims=True)))
    assert np.abs(lp - full[np.arange(B), t]).max() < 2e-5


@pytest.mark.gpu
def test_truncated_sampler_off_equals_plain_and_seeded_draw():
    from ultraviolet_amd.kernels.fused_sample import fused_sample, fused_sample_seeded, sample_filtered
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(64, 4096, generator=g) * 4).bfloat16().to(DEV)
    u = torch.rand(64, generator=g).to(DEV)
    t0, l0 = fused_sample(x, u, SC, 0.9)
    t1, l1 = sample_filtered(x, u, SC, 0.9, 0, 1.0)                      # no filter: the plain kernel runs
    assert torch.equal(t0, t1) and torch.equal(l0, l1)
    t2, l2 = sample_filtered(x, u, SC, 0.9, 4095, 0.9999999)             # a filter that keeps everything
    assert (t0 == t2).float().mean() > 0.98 and (l0 - l2).abs().max() < 2e-5
    req, ti = torch.arange(64, device=DEV), torch.full((64,), 3, device=DEV)
    _, _, us = fused_sample_seeded(x, 7, req, ti, SC, 0.9, return_u=True)
    ta, _ = sample_filtered(x, us, SC, 0.9, 40, 0.8)
    tb, _ = sample_filtered(x, None, SC, 0.9, 40, 0.8, seed=7, req_id=req, tok_idx=ti)
    assert torch.equal(ta, tb)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N", [(5, 640, 656), (128, 640, 3328), (200, 512, 640), (70, 1664, 640), (900, 640, 3328), (515, 1664, 640)])
def test_skinny_gemm_norm_and_resid_fusions(dtype, M, K, N):
    """norm_eps: the product of the RMS-normalised rows, against float64 (rmsnorm(a) @ w.T without intermediate rounding -
    the kernel applies the norm as an exact row scale); RESID: ca * r + cb * round(a @ w.T), rounded; and both with SwiGLU."""
    from ultraviolet_amd.kernels.gemm import RESID, SWIGLU, gemm_tn, interleave_gate_up
    g = torch.Generator(device="cuda").manual_seed(M + N)
    a = (torch.randn(M, K, device="cuda", generator=g) * 3).to(dtype)
    w = (torch.randn(N, K, device="cuda", generator=g) / K ** 0.5).to(dtype)
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    eps = 1e-6
    ad = a.double()
    an = ad * torch.rsqrt((ad * ad).mean(-1, keepdim=True) + eps)
    ref = an @ w.double().t()
    tol = ulp * ref.abs().clamp_min(1.0) + 1e-5 * K ** 0.5
    r = torch.randn(M, N, device="cuda", generator=g).to(dtype)
    prod = (ad @ w.double().t()).to(dtype).double()
    want = 0.75 * r.double() + 1.25 * prod
    tol2 = ulp * want.abs().clamp_min(1.0) + 1.25 * 2 * ulp * prod.abs().clamp_min(1.0)
    for config in (1, 2, 3, 4, 0):
        out = gemm_tn(a, w, norm_eps=eps, config=config)
        assert bool(((out.double() - ref).abs() <= tol).all()), (config, float((out.double() - ref).abs().max()))
        got = gemm_tn(a, w, epilogue=RESID, resid=r, ca=0.75, cb=1.25, config=config)
        assert bool(((got.double() - want).abs() <= tol2).all()), (config, float((got.double() - want).abs().max()))
        inplace = r.clone()       # the residual update in place (C is R), as the engine's output projection runs it
        gemm_tn(a, w, inplace, epilogue=RESID, resid=inplace, ca=0.75, cb=1.25, config=config)
        assert torch.equal(inplace, got)
    if K <= 960 and N % 32 == 0:
        f = N // 2
        wg, wu = w[:f].contiguous(), w[f:].contiguous()
        gg = (an @ wg.double().t()).to(dtype).double()
        uu = (an @ wu.double().t()).to(dtype).double()
        ra = (gg * torch.sigmoid(gg)).to(dtype).double() * uu
        tol3 = 4 * ulp * ra.abs().clamp_min(1.0) + 4 * ulp * (gg.abs() + uu.abs())
        for config in (1, 2, 3, 4, 0):
            act = gemm_tn(a, interleave_gate_up(wg, wu), epilogue=SWIGLU, norm_eps=eps, config=config)
            assert bool(((act.double() - ra).abs() <= tol3).all()), (config, float((act.double() - ra).abs().max()))


@pytest.mark.gpu
def test_tiled_gemm_at_prefill_row_counts():
    """The projections of a packed prefill pass at its size (33 216 rows, the mixed-batch config): gate-up with the pre-norm
    and SwiGLU, and the output projection with the residual update in place, on both tile shapes and on the shape the
    library picks (the 256 x 256 form at this size, config 5), against float64 - thousands of tiles per XCD run, row and
    column tails (33 216 = 259.5 x 128 = 129.75 x 256)."""
    from ultraviolet_amd.kernels.gemm import RESID, SWIGLU, gemm_tn, interleave_gate_up
    dtype, M, K, f = torch.bfloat16, 33216, 640, 1664
    g = torch.Generator(device="cuda").manual_seed(5)
    a = (torch.randn(M, K, device="cuda", generator=g) * 2).to(dtype)
    wg = (torch.randn(f, K, device="cuda", generator=g) / K ** 0.5).to(dtype)
    wu = (torch.randn(f, K, device="cuda", generator=g) / K ** 0.5).to(dtype)
    ulp, eps = 2.0 ** -8, 1e-6
    ad = a.double()
    an = ad * torch.rsqrt((ad * ad).mean(-1, keepdim=True) + eps)
    gg = (an @ wg.double().t()).to(dtype).double()
    uu = (an @ wu.double().t()).to(dtype).double()
    ra = (gg * torch.sigmoid(gg)).to(dtype).double() * uu
    tol = 4 * ulp * ra.abs().clamp_min(1.0) + 4 * ulp * (gg.abs() + uu.abs())
    del an
    for config in (3, 4, 5, 0):
        act = gemm_tn(a, interleave_gate_up(wg, wu), epilogue=SWIGLU, norm_eps=eps, config=config)
        assert bool(((act.double() - ra).abs() <= tol).all()), (config, float((act.double() - ra).abs().max()))
    del gg, uu, ra, tol
    z = (torch.randn(M, 512, device="cuda", generator=g)).to(dtype)
    wo = (torch.randn(K, 512, device="cuda", generator=g) / 512 ** 0.5).to(dtype)
    prod = (z.double() @ wo.double().t()).to(dtype).double()
    want = 0.75 * a.double() + 1.25 * prod
    tol2 = ulp * want.abs().clamp_min(1.0) + 1.25 * 2 * ulp * prod.abs().clamp_min(1.0)
    for config in (3, 4, 5, 0):
        x = a.clone()
        gemm_tn(z, wo, x, epilogue=RESID, resid=x, ca=0.75, cb=1.25, config=config)
        assert bool(((x.double() - want).abs() <= tol2).all()), (config, float((x.double() - want).abs().max()))


@pytest.mark.gpu
def test_gemm_builtin_choice_on_a_head_sized_product():
    """A product of a few thousand rows whose 256 x 256 tiles make several rounds of the device (the tied head of a full decode
    step: 2048 x 32768 x 640) goes to the 256 x 256 form by the built-in choice; with the final norm as its row scale it must
    equal the float64 product of the normalised rows within an ulp of the output type, like the forced forms."""
    from ultraviolet_amd.kernels.gemm import gemm_tn
    dtype, M, K, N = torch.bfloat16, 2048, 640, 32768
    g = torch.Generator(device="cuda").manual_seed(11)
    a = (torch.randn(M, K, device="cuda", generator=g) * 3).to(dtype)
    w = (torch.randn(N, K, device="cuda", generator=g) / K ** 0.5).to(dtype)
    eps, ulp = 1e-6, 2.0 ** -8
    ad = a.double()
    want = (ad * torch.rsqrt((ad * ad).mean(-1, keepdim=True) + eps)) @ w.double().t()
    tol = ulp * want.abs().clamp_min(1.0) + 1e-3
    outs = {}
    for config in (0, 5, 6):
        outs[config] = gemm_tn(a, w, norm_eps=eps, config=config)
        err = (outs[config].double() - want).abs()
        assert bool((err <= tol).all()), (config, float(err.max()))
    assert torch.equal(outs[0], outs[5])   # the built-in choice is the 256 x 256 form here


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N", [(1, 128, 16), (300, 640, 656), (257, 1664, 640), (1000, 512, 640), (700, 640, 3328), (1030, 2048, 224),
                                   (5000, 640, 672), (513, 192, 512)])
def test_big_tile_gemm_matches_float64(dtype, M, K, N):
    """The direct-to-LDS forms (config 5: 256 x 256 tiles, 6: 128 x 128) with every epilogue against float64 on the same 16-bit inputs: ragged M and N (rows
    and weight rows past the end are read clamped and never stored), odd and even slab counts (K / 64), one tile and many,
    padded row pitches, nothing written past column N; to the same bars as the other forms."""
    from ultraviolet_amd.kernels.gemm import RESID, SWIGLU, gemm_tn, interleave_gate_up
    g = torch.Generator(device="cuda").manual_seed(M * 3 + N)
    a = (torch.randn(M, K + 8, device="cuda", generator=g) * 2).to(dtype)[:, :K]
    w = (torch.randn(N, K + 16, device="cuda", generator=g) / K ** 0.5).to(dtype)[:, :K]
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    eps = 1e-6
    ad, wd = a.double(), w.double()
    ref = ad @ wd.t()
    tol = ulp * ref.abs().clamp_min(1.0) + 1e-5 * K ** 0.5
    out_full = torch.full((M, N + 8), 7.0, device="cuda", dtype=dtype)
    an = ad * torch.rsqrt((ad * ad).mean(-1, keepdim=True) + eps)
    refn = an @ wd.t()
    r = torch.randn(M, N, device="cuda", generator=g).to(dtype)
    prod = ref.to(dtype).double()
    want = 0.75 * r.double() + 1.25 * prod
    tol2 = ulp * want.abs().clamp_min(1.0) + 1.25 * 2 * ulp * prod.abs().clamp_min(1.0)
    for config in (5, 6):   # 256 x 256 and 128 x 128 tiles
        out_full = torch.full((M, N + 8), 7.0, device="cuda", dtype=dtype)
        gemm_tn(a, w, out_full[:, :N], config=config)
        assert bool(((out_full[:, :N].double() - ref).abs() <= tol).all()), (config, float((out_full[:, :N].double() - ref).abs().max()))
        assert bool((out_full[:, N:] == 7.0).all())
        out = gemm_tn(a, w, norm_eps=eps, config=config)
        assert bool(((out.double() - refn).abs() <= ulp * refn.abs().clamp_min(1.0) + 1e-5 * K ** 0.5).all()), config
        got = gemm_tn(a, w, epilogue=RESID, resid=r, ca=0.75, cb=1.25, config=config)
        assert bool(((got.double() - want).abs() <= tol2).all()), (config, float((got.double() - want).abs().max()))
        inplace = r.clone()
        gemm_tn(a, w, inplace, epilogue=RESID, resid=inplace, ca=0.75, cb=1.25, config=config)
        assert torch.equal(inplace, got)
    if N % 32 == 0:
        f = N // 2
        wg, wu = w[:f].contiguous(), w[f:].contiguous()
        for nrm, src in ((None, ad), (eps, an)):
            gg = (src @ wg.double().t()).to(dtype).double()
            uu = (src @ wu.double().t()).to(dtype).double()
            ra = (gg * torch.sigmoid(gg)).to(dtype).double() * uu
            tol3 = 4 * ulp * ra.abs().clamp_min(1.0) + 4 * ulp * (gg.abs() + uu.abs())
            for config in (5, 6):
                act_full = torch.full((M, f + 8), 7.0, device="cuda", dtype=dtype)
                gemm_tn(a, interleave_gate_up(wg, wu), act_full[:, :f], epilogue=SWIGLU, norm_eps=nrm, config=config)
                assert bool(((act_full[:, :f].double() - ra).abs() <= tol3).all()), (config, nrm, float((act_full[:, :f].double() - ra).abs().max()))
                assert bool((act_full[:, f:] == 7.0).all())


@pytest.mark.gpu
def test_big_tile_gemm_rejects_what_it_cannot_do():
    """configs 5 and 6 need two K slabs and 16-byte rows of C: asked for anything else they raise instead of running another form."""
    from ultraviolet_amd._lib import UvmiError
    from ultraviolet_amd.kernels.gemm import gemm_tn
    a = torch.randn(300, 128, device="cuda").to(torch.bfloat16)
    w = torch.randn(64, 128, device="cuda").to(torch.bfloat16)
    for config in (5, 6):
        with pytest.raises(UvmiError):
            gemm_tn(a[:, :64], w[:, :64], config=config)                                   # one slab
        with pytest.raises(UvmiError):
            gemm_tn(a, w, torch.empty(300, 68, device="cuda", dtype=torch.bfloat16)[:, :64], config=config)   # pitch 68
        gemm_tn(a, w, config=config)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rope,ring,has_ve,gate", [(1, 1, 1, 1), (0, 0, 0, 1), (1, 1, 0, 0), (1, 0, 1, 1)])
def test_qkv_post_engine_shape_kernel_equals_the_general_kernel(dtype, rope, ring, has_ve, gate):
    """uvmi_qkv_post runs a kernel of its own for the engine's shape (8 heads on 1 kv head, 16 rotated pairs, rotation
    table, logits from the projection, q in the activation type) that requests a row's inputs in two batches.  Asked for
    fp32 queries the same call runs the general kernel; the two must agree bit for bit in everything they write - q (the
    same values), k, v, v_hat, the gates, the appended int8 rows and their scales - on rows inside and past the rotation
    table, rows without a cache row, and a ring that keeps only a prompt's last S positions."""
    import ctypes as C
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels.decode_attn import rope_table
    g = torch.Generator(device="cuda").manual_seed(5 + rope + 2 * ring + 4 * has_ve)
    n, H, S, B, vocab, ld = 333, 8, 64, 40, 500, 656
    qkv = (torch.randn(n, ld, device="cuda", generator=g) * 1.5).to(dtype)
    pos = torch.randint(0, 150, (n,), device="cuda", generator=g)
    rows = torch.randint(-1, B, (n,), device="cuda", generator=g)
    seen, rl = set(), rows.tolist()
    for i, (rw, ps) in enumerate(zip(rl, pos.tolist())):     # no two rows write the same cache slot (the winner would be a race)
        cell = (rw, ps % S if ring else ps)
        if cell in seen:
            rl[i] = -1
        seen.add(cell)
    rows = torch.tensor(rl, device="cuda")
    last = pos + torch.randint(0, 100, (n,), device="cuda", generator=g)
    tok = torch.randint(-3, vocab + 3, (n,), device="cuda", generator=g)     # (out-of-range ids are clamped)
    ve = torch.randn(vocab, 64, device="cuda", generator=g).to(dtype)
    inv_freq = (1.0 / (1024.0 ** (torch.arange(16, device="cuda").float() / 16))).contiguous()
    tab = rope_table(inv_freq, 100, dtype)                                    # positions 100 .. 149 lie past the table
    outs = []
    for qdt in (dtype, torch.float32):
        q = torch.zeros(n, H, 64, device="cuda", dtype=qdt)
        k, v = torch.zeros(n, 64, device="cuda", dtype=dtype), torch.zeros(n, 64, device="cuda", dtype=dtype)
        vhat, gt = torch.zeros(n, 64, device="cuda"), torch.zeros(n, H, device="cuda")
        kc, vc = (torch.zeros(B, 1, S, 64, device="cuda", dtype=torch.int8) for _ in range(2))
        ks, vs = (torch.zeros(B, 1, S, device="cuda", dtype=torch.float16) for _ in range(2))
        a = L.QkvPostArgs()
        a.qkv, a.dtype, a.qkv_ld, a.ext_logits = qkv.data_ptr(), L.dtype_code(dtype), ld, 1
        a.pos, a.rows, a.last_pos, a.inv_freq = pos.data_ptr(), rows.data_ptr(), last.data_ptr() if ring else None, inv_freq.data_ptr()
        if has_ve:
            a.ve_table, a.tok = ve.data_ptr(), tok.data_ptr()
        a.q_out, a.q_dtype, a.k_out, a.v_out = q.data_ptr(), L.dtype_code(qdt), k.data_ptr(), v.data_ptr()
        a.k_cache, a.v_cache, a.k_scale, a.v_scale = kc.data_ptr(), vc.data_ptr(), ks.data_ptr(), vs.data_ptr()
        a.scb, a.sch, a.scs, a.ssb, a.ssh, a.S = kc.stride(0), kc.stride(1), kc.stride(2), ks.stride(0), ks.stride(1), S
        a.n, a.vocab, a.H, a.KH, a.hd, a.d, a.n_pairs = n, vocab, H, 1, 64, 640, 16
        a.ring, a.has_ve, a.rope, a.eps, a.xsa_eps = ring, has_ve, rope, 1e-6, 1e-4
        if rope:
            a.rope_table, a.rope_positions = tab.data_ptr(), tab.size(0)
        a.vhat_out = vhat.data_ptr()
        if gate:
            a.gate_out = gt.data_ptr()
        L.check(L.lib().uvmi_qkv_post(C.byref(a), L.stream_ptr(qkv)), "uvmi_qkv_post")
        torch.cuda.synchronize()
        outs.append((q.float(), k, v, vhat, gt, kc, vc, ks, vs))
    names = ("q", "k", "v", "v_hat", "gate", "k cache", "v cache", "k scale", "v scale")
    for nm, x, y in zip(names, *outs):
        assert torch.equal(x, y), nm
    assert float(outs[0][5].float().abs().sum()) > 0 and float(outs[0][0].abs().sum()) > 0


@pytest.mark.gpu
def test_attention_probe_runs_the_engine_shape_and_refuses_the_rest():
    """uvmi_decode_attn_probe (a measurement aid: the kernel's memory stream without its arithmetic, or the reverse)
    launches for the engine's decode shape, leaves the caches untouched, returns, and refuses other shapes and modes with an
    error instead of running something else.  Its output is meaningless and is not checked."""
    import ctypes as C
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels.decode_attn import build_attn_args
    g = torch.Generator(device="cuda").manual_seed(3)
    B, S = 37, 320
    k, v = (torch.randint(-127, 128, (B, 1, S, 64), device=DEV, dtype=torch.int8, generator=g) for _ in range(2))
    ks, vs = ((torch.rand(B, 1, S, device=DEV, generator=g) * 0.03 + 0.01).half() for _ in range(2))
    q = torch.randn(B, 8, 64, device=DEV, generator=g).bfloat16()
    pos = torch.randint(0, S, (B,), device=DEV, generator=g)
    starts = torch.zeros(B, dtype=torch.long, device=DEV)
    out = torch.zeros_like(q)
    keep = [t.clone() for t in (k, v, ks, vs)]
    stream = torch.cuda.current_stream().cuda_stream
    a, alive = build_attn_args(q, k, v, pos, starts, 0.14125, 0, False, ks, vs, 1, out)
    for mode in (1, 2):
        assert L.lib().uvmi_decode_attn_probe(C.byref(a), mode, stream) == 0, L.lib().uvmi_last_error()
    torch.cuda.synchronize()
    for t, t0 in zip((k, v, ks, vs), keep):
        assert torch.equal(t, t0)
    assert L.lib().uvmi_decode_attn_probe(C.byref(a), 3, stream) != 0                     # no such mode
    a2, alive2 = build_attn_args(q.half(), k, v, pos, starts, 0.14125, 0, False, ks, vs, 1, out.half())
    assert L.lib().uvmi_decode_attn_probe(C.byref(a2), 1, stream) != 0                    # fp16 queries: not the engine's shape
    a3, alive3 = build_attn_args(q, k, v, pos.int(), starts.int(), 0.14125, 0, False, ks, vs, 1, out)
    assert L.lib().uvmi_decode_attn_probe(C.byref(a3), 1, stream) != 0                    # 32-bit indices
    assert b"probe" in L.lib().uvmi_last_error()
