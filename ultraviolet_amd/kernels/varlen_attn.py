"""Packed (cu_seqlens) causal attention with an optional sliding window: host side of uvmi_prefill_attn.

Mirrors ultraviolet/kernels/varlen_attn.py of the reference: the forward (:87-93) on the MFMA kernel, and the backward
(:56-84) in a first, plain form (uvmi_prefill_attn_bwd), wired into autograd as the reference wires its custom ops.
q / k / v must be device tensors; there is no CPU path."""
from __future__ import annotations

import ctypes as C

import torch
from torch import Tensor

from .. import _lib as L


def _args(q, k, v, cu, scale, window, out, ws):
    N, H, hd = q.shape
    a = L.PrefillAttnArgs()
    a.q, a.q_dtype, a.sqn, a.sqh = q.data_ptr(), L.dtype_code(q.dtype), q.stride(0), q.stride(1)
    a.k, a.v, a.kv_dtype = k.data_ptr(), v.data_ptr(), L.dtype_code(k.dtype)
    a.skn, a.skh, a.svn, a.svh = k.stride(0), k.stride(1), v.stride(0), v.stride(1)
    a.cu_seqlens, a.idx_dtype, a.n_seg = cu.data_ptr(), L.dtype_code(cu.dtype), cu.numel() - 1
    a.out, a.out_dtype, a.son, a.soh = out.data_ptr(), L.dtype_code(out.dtype), out.stride(0), out.stride(1)
    a.N, a.H, a.KH, a.hd = N, H, k.size(1), hd
    a.scale, a.window = float(scale), int(window or 0)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    return a


def packed_attention(q: Tensor, k: Tensor, v: Tensor, cu_seqlens: Tensor, scale: float, window: int | None = None,
                     out: Tensor | None = None, out_fp32: bool = False, workspace: Tensor | None = None,
                     segments_ready: bool = False, post: tuple | None = None) -> Tensor:
    """q (N, H, hd) fp16 / bf16, k / v (N, K, hd) (same dtype for the MFMA kernel; fp32 runs the generic kernel),
    cu_seqlens (S+1,) int32 / int64 on the device.  Returns (N, H, hd) in q's dtype (fp32 with out_fp32), or fills `out`.
    `workspace` (uint8, >= uvmi_prefill_attn_workspace_bytes(N)) avoids the allocation; segments_ready: it already holds
    the segment table of these cu_seqlens (an earlier call).  post = (vhat (N, K, hd) fp32, gate (N, H) fp32 or None, xsa
    (H,) fp32 or None) applies Attention.post (XSA, per-head gate; ultraviolet/model.py:321-333) in the kernel's epilogue
    (MFMA kernel only)."""
    L.require_cuda(q, k, v, cu_seqlens)
    assert q.dim() == 3 and k.dim() == 3 and v.shape == k.shape and k.size(0) == q.size(0) and k.size(2) == q.size(2)
    assert q.size(1) % k.size(1) == 0, "H must be a multiple of K"
    assert cu_seqlens.dim() == 1 and cu_seqlens.numel() >= 1 and cu_seqlens.is_contiguous()
    assert v.dtype == k.dtype
    if q.stride(2) != 1:
        q = q.contiguous()
    if k.stride(2) != 1:
        k = k.contiguous()
    if v.stride(2) != 1:
        v = v.contiguous()
    N = q.size(0)
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float32 if out_fp32 else q.dtype, device=q.device)
    assert out.shape == q.shape and out.stride(2) == 1
    if N == 0:
        return out
    need = L.lib().uvmi_prefill_attn_workspace_bytes(N)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    assert workspace.dtype == torch.uint8 and workspace.numel() >= need
    a = _args(q, k, v, cu_seqlens, scale, window, out, workspace)
    a.segments_ready = int(bool(segments_ready))
    if post is not None:
        vhat, gate, xsa = post
        assert vhat.dtype == torch.float32 and vhat.is_contiguous() and vhat.shape == (N, k.size(1), q.size(2))
        a.post_vhat = vhat.data_ptr()
        if gate is not None:
            assert gate.dtype == torch.float32 and gate.is_contiguous() and gate.shape == (N, q.size(1))
            a.post_gate = gate.data_ptr()
        if xsa is not None:
            assert xsa.dtype == torch.float32 and xsa.is_contiguous() and xsa.numel() == q.size(1)
            a.post_xsa = xsa.data_ptr()
    L.check(L.lib().uvmi_prefill_attn(C.byref(a), L.stream_ptr(q)), "uvmi_prefill_attn")
    return out


def packed_attention_path(q: Tensor, k: Tensor, v: Tensor, cu_seqlens: Tensor, scale: float, window: int | None = None) -> int:
    """1 when the MFMA kernel would run for these tensors, 0 for the generic kernel."""
    ws = torch.empty(L.lib().uvmi_prefill_attn_workspace_bytes(q.size(0)), dtype=torch.uint8, device=q.device)
    a = _args(q, k, v, cu_seqlens, scale, window, torch.empty_like(q), ws)
    return int(L.lib().uvmi_prefill_attn_path(C.byref(a)))


def packed_attention_backward(go: Tensor, q: Tensor, k: Tensor, v: Tensor, o: Tensor, cu_seqlens: Tensor, scale: float,
                              window: int | None = None) -> tuple[Tensor, Tensor, Tensor]:
    """(dq, dk, dv) of packed_attention for the output gradient go: q, o, go (N, H, 64), k, v (N, K, 64), one 16-bit dtype
    (reference: mathk::varlen_attn_bwd, varlen_attn.py:56-66; gradients of K / V are summed over the heads of a group)."""
    L.require_cuda(go, q, k, v, o, cu_seqlens)
    assert q.dim() == 3 and k.dim() == 3 and k.shape == v.shape and q.shape == o.shape == go.shape
    assert q.dtype == k.dtype == v.dtype == o.dtype == go.dtype
    assert cu_seqlens.dim() == 1 and cu_seqlens.numel() >= 1 and cu_seqlens.is_contiguous()
    go, q, k, v, o = (t.contiguous() for t in (go, q, k, v, o))
    N, H, hd = q.shape
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ws = torch.empty(L.lib().uvmi_prefill_attn_bwd_workspace_bytes(N, H), dtype=torch.uint8, device=q.device)
    a = L.PrefillAttnBwdArgs(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), go.data_ptr(), L.dtype_code(q.dtype),
                             dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), cu_seqlens.data_ptr(), L.dtype_code(cu_seqlens.dtype),
                             cu_seqlens.numel() - 1, N, H, k.size(1), hd, float(scale), int(window or 0), ws.data_ptr(), ws.numel())
    L.check(L.lib().uvmi_prefill_attn_bwd(C.byref(a), L.stream_ptr(q)), "uvmi_prefill_attn_bwd")
    return dq, dk, dv


class _PackedAttention(torch.autograd.Function):
    """packed_attention with the backward above (the reference registers its pair of custom ops with autograd the same
    way, varlen_attn.py:69-84)."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, scale, window):
        o = packed_attention(q, k, v, cu_seqlens, scale, window)
        ctx.save_for_backward(q, k, v, o, cu_seqlens)
        ctx.scale, ctx.window = scale, window
        return o

    @staticmethod
    def backward(ctx, go):
        q, k, v, o, cu = ctx.saved_tensors
        dq, dk, dv = packed_attention_backward(go, q, k, v, o, cu, ctx.scale, ctx.window)
        return dq, dk, dv, None, None, None


def varlen_attention(q: Tensor, k: Tensor, v: Tensor, cu_seqlens: Tensor, max_seqlen: int, scale: float,
                     window: int | None = None) -> Tensor:
    """The reference's signature: q (1, N, H, hd), k / v (1, N, K, hd) packed along N, cu_seqlens (S+1,) with cu[0] = 0
    and cu[-1] = N; returns (1, N, H, hd).  max_seqlen is accepted for compatibility (the kernel does not need it).
    Differentiable in q, k, v (16-bit inputs, head_dim 64)."""
    assert q.dim() == 4 and q.size(0) == 1 and k.size(0) == 1 and v.size(0) == 1
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        return _PackedAttention.apply(q[0], k[0], v[0], cu_seqlens, float(scale), int(window or 0))[None]
    return packed_attention(q[0], k[0], v[0], cu_seqlens, scale, window)[None]


def _register_reference_ops():
    """mathk::varlen_attn_fwd / mathk::varlen_attn_bwd with the reference's signatures (ultraviolet/kernels/varlen_attn.py:38-84)
    for code that calls the ops directly: q (1, N, H, hd), k / v (1, N, K, hd).  The forward's logsumexp / seed / offset
    outputs exist for the signature only (this backward recomputes the row statistics): they are empty tensors.  Skipped
    when the names are already taken."""
    try:
        @torch.library.custom_op("mathk::varlen_attn_fwd", mutates_args=())
        def fwd(q: Tensor, k: Tensor, v: Tensor, cu: Tensor, max_seqlen: int, window: int, scale: float) -> tuple[Tensor, Tensor, Tensor, Tensor]:
            o = packed_attention(q[0], k[0], v[0], cu, scale, window)[None]
            e = lambda dt: torch.empty(0, dtype=dt, device=q.device)
            return o, e(torch.float32), e(torch.int64), e(torch.int64)

        @fwd.register_fake
        def _(q, k, v, cu, max_seqlen, window, scale):
            e = lambda dt: torch.empty(0, dtype=dt, device=q.device)
            return torch.empty_like(q), e(torch.float32), e(torch.int64), e(torch.int64)

        @torch.library.custom_op("mathk::varlen_attn_bwd", mutates_args=())
        def bwd(go: Tensor, q: Tensor, k: Tensor, v: Tensor, o: Tensor, lse: Tensor, cu: Tensor, seed: Tensor, off: Tensor,
                max_seqlen: int, window: int, scale: float) -> tuple[Tensor, Tensor, Tensor]:
            dq, dk, dv = packed_attention_backward(go[0], q[0], k[0], v[0], o[0], cu, scale, window)
            return dq[None], dk[None], dv[None]

        @bwd.register_fake
        def _(go, q, k, v, o, lse, cu, seed, off, max_seqlen, window, scale):
            return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

        def setup(ctx, inputs, output):
            q, k, v, cu, max_seqlen, window, scale = inputs
            o, lse, seed, off = output
            ctx.save_for_backward(q, k, v, o, lse, cu, seed, off)
            ctx.ms, ctx.window, ctx.scale = max_seqlen, window, scale

        def backward(ctx, go, glse, gseed, goff):
            q, k, v, o, lse, cu, seed, off = ctx.saved_tensors
            dq, dk, dv = bwd(go, q, k, v, o, lse, cu, seed, off, ctx.ms, ctx.window, ctx.scale)
            return dq, dk, dv, None, None, None, None

        fwd.register_autograd(backward, setup_context=setup)
        return fwd, bwd
    except RuntimeError:
        return None


_reference_ops = _register_reference_ops()
