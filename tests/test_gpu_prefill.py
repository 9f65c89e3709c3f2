"""GPU parity: packed causal / windowed prefill attention (uvmi_prefill_attn through the C ABI) vs the CPU oracle.

The first case restates the reference's own test (tests/test_perf_opt.py:40-61, forward part): segment lengths
[300, 1000, 57, 700, 1], 8 query heads on 1 kv head, head_dim 64, fp16, window None / 256, |o - ref|.max() < 2e-3.
With fp16 inputs the probabilities are rounded to fp16 before P.V (as in the reference's tensor-core kernel); with bf16
inputs they are rounded to bf16, which bounds the error by 2^-9 * sum p|v| instead, so that case carries a 4e-3 bar."""
import numpy as np
import pytest
import torch

from util import to_np

pytestmark = pytest.mark.gpu
DEV = "cuda"
SC = 1.13 / 8


def _case(lens, H, K, hd, dtype, seed=0, kv_dtype=None):
    g = torch.Generator().manual_seed(seed)
    N = int(sum(lens))
    q = torch.randn(N, H, hd, generator=g).to(dtype)
    k = torch.randn(N, K, hd, generator=g).to(kv_dtype or dtype)
    v = torch.randn(N, K, hd, generator=g).to(kv_dtype or dtype)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    return q, k, v, cu


def _check(q, k, v, cu, window, atol, expect_path=None, scale=SC):
    from oracle.varlen_attn import varlen_attention_ref
    from ultraviolet_amd.kernels.varlen_attn import packed_attention, packed_attention_path
    d = lambda t: t.to(DEV)
    qd, kd, vd, cud = d(q), d(k), d(v), d(cu)
    if expect_path is not None:
        assert packed_attention_path(qd, kd, vd, cud, scale, window) == expect_path
    o32 = packed_attention(qd, kd, vd, cud, scale, window, out_fp32=True)
    o = packed_attention(qd, kd, vd, cud, scale, window)
    torch.cuda.synchronize()
    ref = varlen_attention_ref(to_np(q), to_np(k), to_np(v), to_np(cu), scale, window)
    a32, a = to_np(o32), to_np(o)
    assert np.isfinite(a32).all()
    assert np.abs(a32 - ref).max() < atol, np.abs(a32 - ref).max()
    out_eps = 2.0 ** -11 if q.dtype == torch.float16 else 2.0 ** -8
    assert np.abs(a - ref).max() < atol + out_eps * np.abs(ref).max()
    return a32, ref


@pytest.mark.parametrize("window", [None, 256])
def test_reference_case_fp16(window):
    q, k, v, cu = _case([300, 1000, 57, 700, 1], 8, 1, 64, torch.float16)
    from ultraviolet_amd.kernels import varlen_attention
    a32, ref = _check(q, k, v, cu, window, 2e-3, expect_path=1)
    o = varlen_attention(q[None].to(DEV), k[None].to(DEV), v[None].to(DEV), cu.to(DEV), 1000, SC, window)
    assert o.shape == (1, q.size(0), 8, 64) and o.dtype == torch.float16
    assert (o[0].float().cpu().numpy() - ref).__abs__().max() < 2e-3   # the reference's bar on the fp16 output


@pytest.mark.parametrize("window", [None, 256])
def test_reference_case_bf16(window):
    q, k, v, cu = _case([300, 1000, 57, 700, 1], 8, 1, 64, torch.bfloat16, seed=1)
    _check(q, k, v, cu, window, 4e-3, expect_path=1)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("lens", [[1], [15], [16], [17], [1, 1, 1, 1, 1], [0, 5, 0, 0, 40, 0], [31, 33, 64, 1, 2, 95, 7],
                                  [512] * 3, [3, 700, 2]])
@pytest.mark.parametrize("window", [None, 1, 16, 33, 256])
def test_ragged_and_edges(dtype, lens, window):
    q, k, v, cu = _case(lens, 8, 1, 64, dtype, seed=len(lens))
    _check(q, k, v, cu, window, 2e-3 if dtype == torch.float16 else 4e-3, expect_path=1)


@pytest.mark.parametrize("H,K", [(1, 1), (4, 1), (5, 1), (8, 2), (6, 2), (16, 2), (8, 8)])
def test_head_groupings(H, K):
    q, k, v, cu = _case([40, 130, 9], H, K, 64, torch.float16, seed=H * 10 + K)
    _check(q, k, v, cu, 64, 2e-3, expect_path=1)


def test_strided_views_of_one_buffer_and_int64_cu():
    """q, k, v as column slices of one (N, (H + 2K) * hd) projection output, as a fused QKV GEMM leaves them."""
    from oracle.varlen_attn import varlen_attention_ref
    from ultraviolet_amd.kernels.varlen_attn import packed_attention, packed_attention_path
    H, K, hd, lens = 8, 1, 64, [100, 37, 260]
    N = sum(lens)
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(N, (H + 2 * K) * hd, generator=g).to(torch.bfloat16).to(DEV)
    q = qkv[:, :H * hd].view(N, H, hd)
    k = qkv[:, H * hd:(H + K) * hd].view(N, K, hd)
    v = qkv[:, (H + K) * hd:].view(N, K, hd)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int64, device=DEV)
    assert packed_attention_path(q, k, v, cu, SC, 256) == 1
    o = packed_attention(q, k, v, cu, SC, 256, out_fp32=True)
    ref = varlen_attention_ref(to_np(q), to_np(k), to_np(v), to_np(cu), SC, 256)
    assert np.abs(to_np(o) - ref).max() < 4e-3


@pytest.mark.parametrize("hd,kv_dtype", [(64, torch.float32), (128, torch.float16), (32, torch.bfloat16)])
def test_generic_path(hd, kv_dtype):
    """fp32 K/V (an fp32 engine keeps q in fp16) and other head dims run the VALU kernel, token by token."""
    qd = torch.float16 if kv_dtype != torch.bfloat16 else torch.bfloat16
    q, k, v, cu = _case([33, 1, 90], 4, 1, hd, qd, seed=3, kv_dtype=kv_dtype)
    _check(q, k, v, cu, 48, 2e-3, expect_path=0, scale=1.0 / np.sqrt(hd))


def test_exact_special_cases():
    """V == 1 gives exactly 1 wherever a row sees any key (sum p~ / sum p, both from the same rounded values up to 2^-11);
    window 1 returns the row's own v (softmax over one key is 1)."""
    from ultraviolet_amd.kernels.varlen_attn import packed_attention
    q, k, v, cu = _case([200, 56, 300], 8, 1, 64, torch.float16, seed=9)
    d = lambda t: t.to(DEV)
    ones = torch.ones_like(v)
    o = packed_attention(d(q), d(k), d(ones), d(cu), SC, 128, out_fp32=True)
    assert np.abs(to_np(o) - 1.0).max() < 1e-3
    o = packed_attention(d(q), d(k), d(v), d(cu), SC, 1, out_fp32=True)
    # p = exp2(fma(s, c, -round(s c))) is 1 up to an ulp, so the normaliser is too
    np.testing.assert_allclose(to_np(o), np.broadcast_to(to_np(v).astype(np.float32), o.shape), rtol=1e-6, atol=0)


@pytest.mark.parametrize("window", [0, 256])
def test_mixed_batch_chunk_shape(window):
    """The prefill half of the mixed-batch configuration: 64 chunks x 512 tokens, bf16, 8 heads on 1 kv head.  The oracle
    checks 3 of the chunks; all chunks see statistically identical inputs, and identical inputs give identical outputs:
    chunk 5 is a copy of chunk 4 shifted by one 512-token (block-aligned) segment, so its output must be bit-identical."""
    from oracle.varlen_attn import varlen_attention_ref
    from ultraviolet_amd.kernels.varlen_attn import packed_attention
    lens = [512] * 64
    q, k, v, cu = _case(lens, 8, 1, 64, torch.bfloat16, seed=11)
    for t in (q, k, v):
        t[5 * 512:6 * 512] = t[4 * 512:5 * 512]
    o = to_np(packed_attention(q.to(DEV), k.to(DEV), v.to(DEV), cu.to(DEV), SC, window, out_fp32=True))
    assert np.isfinite(o).all()
    np.testing.assert_array_equal(o[5 * 512:6 * 512], o[4 * 512:5 * 512])
    for s in (0, 4, 63):
        sl = slice(s * 512, (s + 1) * 512)
        ref = varlen_attention_ref(to_np(q[sl]), to_np(k[sl]), to_np(v[sl]), [0, 512], SC, window)
        assert np.abs(o[sl] - ref).max() < 4e-3


def test_error_paths():
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels.varlen_attn import packed_attention
    q, k, v, cu = _case([20], 8, 1, 64, torch.float16)
    with pytest.raises(L.UvmiError):
        packed_attention(q, k, v, cu, SC)                       # host tensors
    d = lambda t: t.to(DEV)
    with pytest.raises((L.UvmiError, KeyError)):
        packed_attention(d(q).double(), d(k), d(v), d(cu), SC)   # queries are fp16, bf16 or fp32
    o32 = packed_attention(d(q).float(), d(k).float(), d(v).float(), d(cu), SC)   # fp32 throughout: the plain fp32 kernel
    o16 = packed_attention(d(q), d(k), d(v), d(cu), SC, out_fp32=True)
    assert o32.dtype == torch.float32 and (o32 - o16).abs().max() < 2e-3
    with pytest.raises(AssertionError):
        packed_attention(d(q), d(k), d(v), d(cu), SC, workspace=torch.empty(64, dtype=torch.uint8, device=DEV))  # too small


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 48])
def test_packed_attention_fused_post_epilogue(dtype, window):
    """post=(vhat, gate, xsa): the kernel's epilogue equals Attention.post applied to its own plain output
    (ultraviolet/model.py:321-333: z -= xsa_h (z . v_hat) v_hat on the output rounded to the activation type, then the
    per-head gate), evaluated here in float64 from the plain output of the same kernel; reusing the segment table of an
    earlier call (segments_ready) changes nothing."""
    from ultraviolet_amd.kernels.varlen_attn import packed_attention
    g = torch.Generator(device="cuda").manual_seed(5)
    lens = [37, 1, 160, 64, 5]
    N, H, K, hd = sum(lens), 8, 2, 64
    cu = torch.tensor([0] + list(np.cumsum(lens)), device="cuda")
    q = torch.randn(N, H, hd, device="cuda", generator=g).to(dtype)
    k = torch.randn(N, K, hd, device="cuda", generator=g).to(dtype)
    v = torch.randn(N, K, hd, device="cuda", generator=g).to(dtype)
    vhat = torch.nn.functional.normalize(v.float(), dim=-1).contiguous()
    gate = (torch.rand(N, H, device="cuda", generator=g) * 2).contiguous()
    xsa = torch.tanh(torch.randn(H, device="cuda", generator=g)).contiguous()
    ws = torch.empty(1 << 16, dtype=torch.uint8, device="cuda")
    plain = packed_attention(q, k, v, cu, 0.125, window, workspace=ws)
    fused = packed_attention(q, k, v, cu, 0.125, window, workspace=ws, segments_ready=True, post=(vhat, gate, xsa))
    z = plain.double()
    vh = vhat.double().repeat_interleave(H // K, dim=1)
    want = (z - xsa.double()[None, :, None] * (z * vh).sum(-1, keepdim=True) * vh) * gate.double()[:, :, None]
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    err = (fused.double() - want).abs()
    assert float((err / (want.abs() + 1.0)).max()) <= 3 * ulp, float((err / (want.abs() + 1.0)).max())
    no_gate = packed_attention(q, k, v, cu, 0.125, window, workspace=ws, post=(vhat, None, None))
    assert float((no_gate.double() - z).abs().max()) <= 2 * ulp * float(z.abs().max())


def _grad_case(lens, H, K, dtype, window, seed=0):
    from oracle.varlen_attn import varlen_attention_grad_ref
    from ultraviolet_amd.kernels import varlen_attention
    q, k, v, cu = _case(lens, H, K, 64, dtype, seed=seed)
    go = torch.randn(q.shape, generator=torch.Generator().manual_seed(seed + 100)).to(dtype)
    qd, kd, vd = (t[None].to(DEV).requires_grad_() for t in (q, k, v))
    o = varlen_attention(qd, kd, vd, cu.to(DEV), max(max(lens), 1), SC, window)
    o.backward(go[None].to(DEV))
    torch.cuda.synchronize()
    ref = varlen_attention_grad_ref(to_np(q), to_np(k), to_np(v), to_np(go), to_np(cu), SC, window)
    got = [to_np(t.grad[0]).astype(np.float64) for t in (qd, kd, vd)]
    return got, ref


@pytest.mark.parametrize("window", [None, 256])
def test_backward_reference_case_fp16(window):
    """The reference's own test of the varlen backward (tests/test_perf_opt.py:40-61): lens [300, 1000, 57, 700, 1], 8 query
    heads on 1 kv head, fp16, window None / 256, gradients through autograd; its bar: |g - g_ref| / |g_ref| < 5e-3 for each
    of dq, dk, dv (norms over the whole tensor)."""
    got, ref = _grad_case([300, 1000, 57, 700, 1], 8, 1, torch.float16, window)
    for a, b in zip(got, ref):
        assert np.isfinite(a).all()
        assert np.linalg.norm(a - b) / np.linalg.norm(b) < 5e-3, np.linalg.norm(a - b) / np.linalg.norm(b)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("lens,H,K,window", [([1], 8, 1, None), ([0, 5, 0, 0, 40, 0], 8, 1, 16), ([31, 33, 64, 1, 2, 95, 7], 8, 2, 33),
                                             ([70, 3], 4, 4, 1), ([130], 2, 1, None), ([65, 64, 63], 8, 8, 64)])
def test_backward_ragged_and_edges(dtype, lens, H, K, window):
    """Empty and single-token segments, segment boundaries inside a wave's 64 queries / 32 keys, window 1 (every query sees
    only itself: dq = dk = 0 up to rounding, dv = go summed over the group), grouped and per-head K / V."""
    got, ref = _grad_case(lens, H, K, dtype, window, seed=3)
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    for a, b in zip(got, ref):
        assert np.isfinite(a).all()
        assert np.abs(a - b).max() <= 2 * ulp * max(np.abs(b).max(), 1e-3) + 1e-6, (np.abs(a - b).max(), np.abs(b).max())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,K,window", [(8, 1, None), (8, 2, 256), (4, 1, 100), (16, 1, 64)])
def test_backward_many_tiles_and_padding_tokens(dtype, H, K, window):
    """Sequences of several 32-key tiles and 64-key workgroups (interior tiles take the unmasked path), a group of 16 heads
    (beyond the matrix-core kernels' 8: the plain kernels), and 37 tokens past cu[-1]: padding, whose gradients are zero and
    which no real key may see."""
    from oracle.varlen_attn import varlen_attention_grad_ref
    from ultraviolet_amd.kernels.varlen_attn import packed_attention, packed_attention_backward
    lens, pad = [512, 700, 300, 5], 37
    q, k, v, cu = _case(lens, H, K, 64, dtype, seed=11)
    N = q.size(0)
    gen = torch.Generator().manual_seed(12)
    go = torch.randn(q.shape, generator=gen).to(dtype)
    ext = lambda t: torch.cat([t, torch.randn(pad, *t.shape[1:], generator=gen).to(dtype)]).to(DEV)
    qd, kd, vd, god = ext(q), ext(k), ext(v), ext(go)
    o = packed_attention(qd, kd, vd, cu.to(DEV), SC, window)
    dq, dk, dv = packed_attention_backward(god, qd, kd, vd, o, cu.to(DEV), SC, window)
    torch.cuda.synchronize()
    ref = varlen_attention_grad_ref(to_np(q), to_np(k), to_np(v), to_np(go), to_np(cu), SC, window)
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    for a, b in zip((dq, dk, dv), ref):
        a = to_np(a).astype(np.float64)
        assert np.isfinite(a).all() and (a[N:] == 0).all()
        assert np.abs(a[:N] - b).max() <= 2 * ulp * np.abs(b).max() + 1e-6, (np.abs(a[:N] - b).max(), np.abs(b).max())
        assert np.linalg.norm(a[:N] - b) / np.linalg.norm(b) < (5e-3 if dtype == torch.float16 else 2e-2)


def test_backward_rejects_what_it_cannot_do():
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels.varlen_attn import packed_attention_backward
    cu = torch.tensor([0, 4], dtype=torch.int32, device=DEV)
    z = lambda *s_, dt=torch.float16: torch.zeros(*s_, dtype=dt, device=DEV)
    with pytest.raises(L.UvmiError):   # head_dim 32
        packed_attention_backward(z(4, 2, 32), z(4, 2, 32), z(4, 1, 32), z(4, 1, 32), z(4, 2, 32), cu, 1.0)
    with pytest.raises(L.UvmiError):   # fp32 tensors
        packed_attention_backward(*(z(4, 2, 64, dt=torch.float32) for _ in range(2)), *(z(4, 1, 64, dt=torch.float32) for _ in range(2)),
                                  z(4, 2, 64, dt=torch.float32), cu, 1.0)
