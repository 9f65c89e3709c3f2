"""Fused softcap + categorical sample + behaviour log-prob for the decode step (one kernel), with either caller
uniforms or in-kernel Philox4x32-10 keyed by (seed, request id, token index).

Mirror of ultraviolet/kernels/fused_sample.py of the reference; the kernel is in csrc/fused_sample.hip."""
from __future__ import annotations

import ctypes as C

import torch
from torch import Tensor

from .. import _lib as L

BLOCK = 512  # the kernel's chunk; V must be a multiple of it and V / BLOCK <= 64


def fused_sample_ok(x_or_dev, V: int, softcap, temperature: float, block: int = BLOCK) -> bool:
    """When the fused sampler applies (reference: fused_sample.py:61-65): a GPU device, V a multiple of the chunk with at
    most 64 chunks, T > 0 and a / T small enough for the bounded exp in fp32."""
    dev = x_or_dev.device if isinstance(x_or_dev, Tensor) else torch.device(x_or_dev)
    a = float(softcap[0])
    return bool(dev.type == "cuda" and V % block == 0 and V // block <= 64 and temperature > 0
                and a / temperature <= 80.0)


def _run(x, u, softcap, temperature, seed, req_id, tok_idx, want_u, top_k=0, top_p=1.0, want_thr=False, commit=None):
    L.require_cuda(x, u, req_id, tok_idx)
    B, V = x.shape
    assert x.stride(1) == 1 and V % BLOCK == 0
    tok = torch.empty(B, dtype=torch.int64, device=x.device)
    lp = torch.empty(B, dtype=torch.float32, device=x.device)
    uo = torch.empty(B, dtype=torch.float32, device=x.device) if want_u else None
    a, b, c = (float(v) for v in softcap)
    s = L.SampleArgs(x.data_ptr(), L.dtype_code(x.dtype), x.stride(0), None if u is None else u.data_ptr(),
                     int(seed) & (2 ** 64 - 1), None if req_id is None else req_id.data_ptr(),
                     None if tok_idx is None else tok_idx.data_ptr(), tok.data_ptr(), lp.data_ptr(),
                     None if uo is None else uo.data_ptr(), B, V, a, b, c, float(temperature), int(top_k), float(top_p),
                     None, None)
    if commit is not None:   # an _lib.SampleCommit: the launch also commits the rows' tokens to the slot table
        s.commit = C.addressof(commit)
    thr = None
    if want_thr:
        thr = torch.zeros(B, dtype=torch.float32, device=x.device)
        s.thr_out = thr.data_ptr()
    L.check(L.lib().uvmi_fused_sample(C.byref(s), L.stream_ptr(x)), "uvmi_fused_sample")
    return (tok, lp, uo, thr) if want_thr else (tok, lp, uo)


def fused_sample(x: Tensor, u: Tensor, softcap, temperature: float = 1.0, block: int = BLOCK) -> tuple[Tensor, Tensor]:
    """x (B, V) fp16/bf16/fp32 raw head output (before the softcap), u (B,) fp32 uniforms in [0, 1) -> (tokens int64
    (B,), log softmax(softcap(x) / T)[token] fp32 (B,)).  Graph-capturable (no host syncs).
    (reference: fused_sample.py:68-77)"""
    assert u.dtype == torch.float32 and u.is_contiguous() and u.numel() == x.size(0)
    tok, lp, _ = _run(x, u, softcap, temperature, 0, None, None, False)
    return tok, lp


def fused_sample_seeded(x: Tensor, seed: int, req_id: Tensor, tok_idx: Tensor, softcap, temperature: float = 1.0,
                        return_u: bool = False, top_k: int = 0, top_p: float = 1.0, commit=None):
    """Same draw with u = Philox4x32-10(key = seed, counter = (tok_idx, req_id, "SAMP")) generated in the kernel:
    replaces the torch.rand(B) feeding the reference's sampler (ultraviolet/perf.py:595) with a stream keyed by request
    and token index, so it does not depend on slot placement.  req_id, tok_idx: (B,) int64.  top_k / top_p truncate the
    distribution as sample() does (model.py:1200-1209; see sample_filtered).  commit (an _lib.SampleCommit): the rows are the
    dense rows of a decode step and the launch also commits their tokens to the slot table (uvmi_sched_commit_dense)."""
    assert req_id.dtype == torch.int64 and tok_idx.dtype == torch.int64
    tok, lp, uo = _run(x, None, softcap, temperature, seed, req_id.contiguous(), tok_idx.contiguous(), return_u, top_k, top_p, commit=commit)
    return (tok, lp, uo) if return_u else (tok, lp)


def greedy_sample(x: Tensor, softcap, commit=None) -> tuple[Tensor, Tensor]:
    """argmax (first maximal index) of the head output and log softmax(softcap(x))[argmax]: the T <= 0 branch of the
    reference's sample() (ultraviolet/model.py:1198-1199) fused with the log-prob.  commit: as in fused_sample_seeded."""
    tok, lp, _ = _run(x, None, softcap, 0.0, 0, None, None, False, commit=commit)
    return tok, lp


def sample_filtered(x: Tensor, u: Tensor | None, softcap, temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0, *,
                    seed: int = 0, req_id: Tensor | None = None, tok_idx: Tensor | None = None, return_threshold: bool = False):
    """Top-k / nucleus sampling of the reference's sample() (ultraviolet/model.py:1194-1211) fused with the softcap and the
    behaviour log-prob: tokens below the k-th largest value are dropped, then the smallest prefix by probability whose mass
    reaches top_p is kept, and the token is drawn from what is left by inverse CDF with u (or, u=None, with the Philox
    uniform of (seed, req_id, tok_idx)).  logp is log softmax(softcap(x) / T)[token], untruncated (model.py:1161-1169).
    return_threshold adds the smallest kept exp((z - a) / T) per row."""
    assert temperature > 0
    if u is not None:
        assert u.dtype == torch.float32 and u.is_contiguous() and u.numel() == x.size(0)
    else:
        assert req_id is not None and tok_idx is not None and req_id.dtype == torch.int64 and tok_idx.dtype == torch.int64
    out = _run(x, u, softcap, temperature, seed, None if req_id is None else req_id.contiguous(),
               None if tok_idx is None else tok_idx.contiguous(), False, top_k, top_p, return_threshold)
    return (out[0], out[1], out[3]) if return_threshold else (out[0], out[1])
