"""uvmi_decode_attn_noalloc through the C ABI: the split-K decode attention whose partials live in the library's own
device array instead of a caller's workspace.  Its output must equal uvmi_decode_attn's (same kernels, same partials) bit
for bit, on two calls in a row - the second smaller, so that it runs over what the first left in the array - and it must
refuse what does not fit.  Collected last: it shares one device array with whatever ran before it."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(B, S, seed, dtype=torch.bfloat16):
    from oracle import kv_quant as okv
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    k, v = torch.randn(B, 1, S, 64, generator=g), torch.randn(B, 1, S, 64, generator=g)
    kq, ks = okv.quantize_kv(k.numpy())
    vq, vs = okv.quantize_kv(v.numpy())
    q = torch.randn(B, 8, 64, generator=g).to(dtype)
    pos = rng.integers(0, S, size=B)
    starts = np.where(rng.random(B) < 0.3, rng.integers(0, S, size=B) % (pos + 1), 0)
    d = lambda a: torch.as_tensor(a).to(DEV)
    return dict(q=q.to(DEV), kq=d(kq), vq=d(vq), ks=d(ks), vs=d(vs), pos=d(pos), starts=d(starts),
                np=(q.float().numpy(), kq, vq, ks, vs, pos, starts))


def _both(c, splits, out_dtype=torch.float32):
    """(uvmi_decode_attn with a workspace, uvmi_decode_attn_noalloc) on the same arguments."""
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels.decode_attn import build_attn_args
    outs = []
    for entry in ("uvmi_decode_attn", "uvmi_decode_attn_noalloc"):
        out = torch.full(c["q"].shape, float("nan"), dtype=out_dtype, device=DEV)
        a, keep = build_attn_args(c["q"], c["kq"], c["vq"], c["pos"], c["starts"], 0.14125, 0, False, c["ks"], c["vs"], splits, out)
        if entry.endswith("noalloc"):
            a.workspace, a.workspace_bytes = None, 0          # the entry point must not need it
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        rc = getattr(L.lib(), entry)(C.byref(a), L.stream_ptr(out))
        L.check(rc, entry)
        assert torch.cuda.memory_allocated() == before        # nothing through torch's allocator
        torch.cuda.synchronize()
        if entry.endswith("noalloc") and _both.calls > 0:      # and nothing through hipMalloc either (the driver's free bytes;
            assert torch.cuda.mem_get_info()[0] == free_before  # the first call on a device may look the scratch symbol up)
        if entry.endswith("noalloc"):
            _both.calls += 1
        outs.append(out.cpu())
        del keep
    return outs


_both.calls = 0


def test_noalloc_entry_matches_workspace_entry_twice_and_smaller():
    from oracle import decode_attn as odec
    big, small = _case(192, 1024, 1), _case(40, 512, 2)
    for c, splits in ((big, 4), (small, 3)):                  # the second call is smaller and reuses the array as it was left
        ws, na = _both(c, splits)
        assert torch.isfinite(na).all()
        assert torch.equal(ws.view(torch.int32), na.view(torch.int32))
        qf, kq, vq, ks, vs, pos, starts = c["np"]
        ref = odec.decode_attention_ref(qf, kq, vq, pos, starts, 0.14125, k_scale=ks, v_scale=vs)
        np.testing.assert_allclose(na.numpy(), ref, atol=2e-3, rtol=2e-3)
    ws, na = _both(small, 2, torch.bfloat16)                  # a 16-bit output through the combine pass as well
    assert torch.equal(ws.view(torch.int16), na.view(torch.int16))
    ws, na = _both(big, 1)                                    # one chunk per row: no partials, no scratch
    assert torch.equal(ws.view(torch.int32), na.view(torch.int32))


def test_noalloc_entry_refuses_what_exceeds_its_scratch():
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels.decode_attn import build_attn_args
    c = _case(512, 64, 3)
    splits = 64
    need = L.lib().uvmi_decode_attn_workspace_bytes(512, 8, 1, 64, splits)
    assert need > (8 << 20)
    out = torch.zeros(c["q"].shape, dtype=torch.float32, device=DEV)
    a, keep = build_attn_args(c["q"], c["kq"], c["vq"], c["pos"], c["starts"], 0.14125, 0, False, c["ks"], c["vs"], splits, out)
    rc = L.lib().uvmi_decode_attn_noalloc(C.byref(a), L.stream_ptr(out))
    assert rc == -3                                           # UVMI_EWORKSPACE
    msg = L.lib().uvmi_last_error().decode()
    assert "built-in scratch" in msg and str(need) in msg
    torch.cuda.synchronize()
    assert float(out.abs().max()) == 0.0                      # nothing was launched
