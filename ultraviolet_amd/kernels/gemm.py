"""Skinny 16-bit GEMM of a small decode step's projections (uvmi_gemm_tn): out = a @ w.T with fp32 accumulation,
optionally with the SwiGLU of the MLP folded into the epilogue.  Stands in for the F.linear calls of the reference's
fused inference path (ultraviolet/model.py:302-335, 388-391) when the batch is a few hundred rows."""
from __future__ import annotations

import ctypes as C

import torch
from torch import Tensor

from .. import _lib as L

STORE, SWIGLU, RESID = 0, 1, 2


def gemm_supported(a: Tensor, w: Tensor, epilogue: int = STORE) -> bool:
    if not (a.is_cuda and a.dim() == 2 and w.dim() == 2 and a.dtype == w.dtype and a.dtype in (torch.float16, torch.bfloat16)):
        return False
    if a.stride(1) != 1 or w.stride(1) != 1 or a.size(1) != w.size(1) or a.data_ptr() % 16 or w.data_ptr() % 16:
        return False
    n_out = w.size(0) // 2 if epilogue == SWIGLU else w.size(0)
    return bool(L.lib().uvmi_gemm_tn_supported(L.dtype_code(a.dtype), a.size(0), w.size(0), a.size(1), a.stride(0), w.stride(0),
                                               n_out, epilogue))


def gemm_tn(a: Tensor, w: Tensor, out: Tensor | None = None, epilogue: int = STORE, *, norm_eps: float | None = None,
            resid: Tensor | None = None, ca: float = 1.0, cb: float = 1.0, config: int = 0) -> Tensor:
    """a (M, K) @ w (N, K).T -> (M, N); with epilogue=SWIGLU w is interleave_gate_up(w_gate, w_up) and the result is
    silu(a @ w_gate.T) * (a @ w_up.T), (M, N / 2); with epilogue=RESID the result is ca * resid + cb * (a @ w.T) (the
    block's residual update, ultraviolet/model.py:567-571).  norm_eps: a stands for rmsnorm(a) with that epsilon (the
    pre-norm of the block folded into the projection as a row scale of the product).  Raises UvmiError for shapes the
    kernel does not take.  config (tuning / tests): 0 built-in choice, 1 the 64-row workgroup form, 2 the 16-row form whose
    waves split K."""
    M, K = a.shape
    N = w.size(0)
    n_out = N // 2 if epilogue == SWIGLU else N
    if out is None:
        out = torch.empty(M, n_out, dtype=a.dtype, device=a.device)
    assert out.shape == (M, n_out) and out.dtype == a.dtype and out.stride(1) == 1 and a.stride(1) == 1 and w.stride(1) == 1
    g = L.GemmArgs(a.data_ptr(), w.data_ptr(), out.data_ptr(), L.dtype_code(a.dtype), M, N, K, a.stride(0), w.stride(0), out.stride(0),
                   epilogue, 0 if norm_eps is None else 1, 0.0 if norm_eps is None else float(norm_eps), None, 0, float(ca), float(cb), int(config))
    if epilogue == RESID:
        assert resid is not None and resid.shape == (M, N) and resid.dtype == a.dtype and resid.stride(1) == 1
        g.resid, g.ldr = resid.data_ptr(), resid.stride(0)
    L.check(L.lib().uvmi_gemm_tn_ex(C.byref(g), L.stream_ptr(a)), "uvmi_gemm_tn")
    return out


def interleave_gate_up(w_gate: Tensor, w_up: Tensor) -> Tensor:
    """(f, K), (f, K) -> (2 f, K) in slabs of 16 rows [gate 0..15 | up 0..15 | gate 16..31 | ...]: the weight layout of the
    SWIGLU epilogue (f % 16 == 0)."""
    f, K = w_gate.shape
    assert w_up.shape == (f, K) and f % 16 == 0
    return torch.stack([w_gate.view(f // 16, 16, K), w_up.view(f // 16, 16, K)], 1).reshape(2 * f, K).contiguous()
