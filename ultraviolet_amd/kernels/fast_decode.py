"""Model-level mirror of ultraviolet/kernels/fast_decode.py: the names a caller of the reference's kernel decode path
uses (KernelDecodeState, prefill_fast, decode_step_fast, patch_model, unpatch_model, kv_bytes_per_seq), backed by the
UV engine of this package.  patch_model(model) reads model.cfg and model.state_dict() (the reference's MathLM: same field
and parameter names), builds the fused device weights once, and binds new_state / prefill / decode_step onto the
instance exactly as the reference's patch_model does (fast_decode.py:341-364); the model's own forward is untouched.

kv_dtype "int8" (the fast path) or "fp16" (unquantized, in the engine's 16-bit dtype); attention-only presets (uv-50m-alpha) only."""
from __future__ import annotations

import types

import numpy as np
import torch
from torch import Tensor

from .. import _lib as L
from ..engine.config import UVConfig
from ..engine.config import as_uvconfig as _as_uvconfig
from ..engine.model import KVState, UVEngine
from ..engine.model import kv_bytes_per_seq as _kv_bytes
from ..engine.weights import UVWeights


def as_uvconfig(cfg) -> UVConfig:
    """engine.config.as_uvconfig with this module's error type."""
    try:
        return _as_uvconfig(cfg)
    except ValueError as e:
        raise L.UvmiError(str(e)) from None


class KernelDecodeState(KVState):
    """KernelDecodeState(cfg, B, max_len, dtype, device, kv_dtype) of the reference (fast_decode.py:21-57): per-layer
    k / v (B, K, S, hd) int8 and k_scale / v_scale (B, K, S) fp16, S = max_len on global layers (rounded up to a
    multiple of 32 here) and min(window, max_len) on local ones, plus pos / starts / host_pos."""

    def __init__(self, cfg, B: int, max_len: int, dtype=torch.float16, device="cuda", kv_dtype: str = "int8"):
        if kv_dtype not in ("int8", "fp16"):
            raise L.UvmiError(f"kv_dtype {kv_dtype!r}: the KV layouts are 'int8' and 'fp16' (unquantized, in the compute dtype)")
        super().__init__(as_uvconfig(cfg), B, max_len, device, kv_dtype=kv_dtype, dtype=dtype)
        self.dtype = dtype
        self.host_pos = np.zeros(B, dtype=np.int64)


class DecodeState(KVState):
    """DecodeState(cfg, B, max_len, dtype, device) of the reference (ultraviolet/model.py:1042-1072): the uncompressed cache
    of its SDPA decode path - k[l], v[l] (B, K, S, hd) in `dtype`, S = max_len on global layers (rounded up to a multiple of
    32 here) and min(window, max_len) ring slots on local ones, pos / starts (B,) int64 on the device, host_pos, kv_dtype =
    None, set_pos, nbytes.  Where the reference attends such a cache through dense additive masks over all g_len slots
    (model.py:968-1002), the engine reads each row's valid range lo..pos from it - the same keys.  16-bit dtypes."""
    mix: dict = {}
    prev = None

    def __init__(self, cfg, B: int, max_len: int, dtype=torch.bfloat16, device="cuda"):
        if dtype not in (torch.float16, torch.bfloat16):
            raise L.UvmiError("DecodeState keeps K / V in a 16-bit dtype (the engine's activation type)")
        super().__init__(as_uvconfig(cfg), B, max_len, device, kv_dtype="fp16", dtype=dtype)
        self.kv_dtype = None          # the reference's marker of the uncompressed state (model.py:1045)
        self.dtype = dtype
        self.host_pos = np.zeros(B, dtype=np.int64)

    def set_pos(self, p: int):
        self.pos.fill_(p)
        self.host_pos[:] = p


def kv_bytes_per_seq(cfg, ctx: int, kv_dtype: str = "int8") -> int:
    """Cache bytes of one sequence at context ctx (reference: fast_decode.py:60-67): hd + 2 bytes per key / value row
    with int8 + fp16 scale, 2 hd unquantized."""
    c = as_uvconfig(cfg)
    if kv_dtype == "int8":
        return _kv_bytes(c, ctx)
    return sum(2 * c.n_kv_heads * 2 * c.head_dim * (ctx if c.is_global(l) else min(ctx, c.window)) for l in range(c.n_layers))


def _live_tensors(model) -> dict:
    """The model's parameters and buffers as the objects the model itself holds.  nn.Module.state_dict() hands out fresh
    detached tensors on every call (their ids never repeat); keep_vars=True returns the live ones, whose storage address and
    version counter identify the weights.  Objects whose state_dict takes no such argument (a plain dict of tensors behind a
    state_dict() method) hold their tensors directly."""
    try:
        return dict(model.state_dict(keep_vars=True))
    except TypeError:
        return dict(model.state_dict())


def _weights_stamp(model) -> tuple:
    """Changes whenever a parameter of the model was written in place or replaced: (name, storage address, version counter)
    of every live tensor (torch bumps the counter on every in-place write - optimizer steps, copy_, the parameter copy of
    scripts/rl_stream.py:22-36).  Stable across calls when nothing was written."""
    return tuple((k, t.data_ptr(), t._version) for k, t in _live_tensors(model).items())


def _quick_stamp(model) -> tuple:
    """The version counters of the tensors seen by the last full stamp: what a decode step checks (a few dozen attribute
    reads, no state_dict walk).  Replaced parameter objects are caught by the full stamp of the next prefill / chunk."""
    return tuple(t._version for t in model.__dict__.get("_uvmi_live", ()))


def _remember_stamp(model) -> None:
    live = _live_tensors(model)
    model.__dict__["_uvmi_live"] = tuple(live.values())
    model.__dict__["_uvmi_stamp"] = tuple((k, t.data_ptr(), t._version) for k, t in live.items())
    model.__dict__["_uvmi_quick"] = tuple(t._version for t in live.values())


def _engine(model, full_check: bool = True) -> UVEngine:
    """The engine bound to a patched model, with its fused device weights brought up to date first: the reference's patched
    methods read the model's live fused weights (fast_decode.py:296-311), so a caller that updates the parameters in place
    expects the next prefill / decode step to use them.  full_check: walk state_dict (prefill, a generator's chunk);
    otherwise only the version counters of the tensors seen by the last walk are compared (every decode step)."""
    eng = model.__dict__.get("_uvmi_engine")
    if eng is None:
        raise L.UvmiError("model has not been patched: call patch_model(model) first")
    if full_check:
        stale = _weights_stamp(model) != model.__dict__.get("_uvmi_stamp")
    else:
        stale = _quick_stamp(model) != model.__dict__.get("_uvmi_quick")
    if stale:
        sync_patched_weights(model)
    return eng


@torch.no_grad()
def prefill_fast(self, idx: Tensor, starts: Tensor, st: KVState, rows: Tensor | None = None) -> Tensor:
    """idx (n, T) left-padded prompts, starts (n,) first real column of each; writes the int8 caches of `rows` (all
    rows when None), sets st.pos = T and st.starts = starts, returns the softcapped fp32 logits of the last position
    (fast_decode.py:70-115).  Runs packed: pad columns are never computed."""
    eng = _engine(self)
    n, T = idx.shape
    assert T <= st.max_len
    if rows is None:
        assert n == st.B
        rows_l = list(range(n))
    else:
        rows_l = [int(r) for r in rows.tolist()]
    idx_h, st_h = idx.cpu().numpy(), starts.cpu().numpy()
    prompts = [idx_h[b, int(st_h[b]):].tolist() for b in range(n)]
    assert max(len(p) for p in prompts) == T, "the longest prompt must fill all T columns (left padding)"
    h = eng.prefill(prompts, rows_l, st, left_pad=True)
    if hasattr(st, "host_pos"):
        st.host_pos[np.asarray(rows_l)] = T
    return eng.logits(h)


@torch.no_grad()
def prefill_packed_host(self, prompts, rows, st: KVState, dev=None) -> Tensor:
    """prompts (lists of token ids) prefilled into cache rows `rows` with every index table built on the host from the
    prompt lengths - the reference's perf flag 'rfh' (fast_decode.py:210-269), which StreamGen's _refill_host calls
    (ultraviolet/perf.py:620-648).  Left-padded positions (token j of a prompt of length n at T - n + j, T the longest
    prompt of the call), so cache slots, st.pos / starts / host_pos and the returned logits of each prompt's last token
    equal prefill_fast's on the left-padded batch.  `dev` is accepted for the reference's signature."""
    eng = _engine(self)
    rows_l = [int(r) for r in rows]
    T = max(len(p) for p in prompts)
    assert T <= st.max_len
    h = eng.prefill([list(p) for p in prompts], rows_l, st, left_pad=True)
    if hasattr(st, "host_pos"):
        st.host_pos[np.asarray(rows_l)] = T
    return eng.logits(h)


@torch.no_grad()
def decode_step_fast(self, tok: Tensor, st: KVState, g_len: int = 0, skip_attn: bool = False, num_splits: dict | None = None,
                     backend: str = "auto", return_hidden: bool = False) -> Tensor:
    """One token for all rows at st.pos, then st.pos += 1 (fast_decode.py:272-334).  g_len is accepted and ignored: the
    kernels take every row's valid range from st.pos / st.starts.  Returns the logits, or the final normed hidden with
    return_hidden (the caller then runs the head GEMM and the fused sampler)."""
    assert not skip_attn, "skip_attn is a profiling switch of the reference and is not supported"
    assert backend in ("auto", "hip"), f"backend {backend!r}: this library has one backend"
    eng = _engine(self, full_check=False)
    h = eng.decode_step(tok, st, num_splits)
    if hasattr(st, "host_pos"):
        st.host_pos += 1
    return h if return_hidden else eng.logits(h)


def patch_model(model, kv_dtype: str | None = "fp16", num_splits: dict | None = None, backend: str = "auto",
                dtype: torch.dtype = torch.bfloat16, max_tokens: int = 16384, device=None):
    """Bind the kernel decode path onto `model` (instance attributes only).  model.cfg and model.state_dict() must use
    the reference's names.  dtype: activation / weight dtype of the engine; max_tokens: largest number of token rows of
    one call (decode rows or packed prefill tokens).  kv_dtype None (or "sdpa") binds the reference's uncompressed
    DecodeState instead of a KernelDecodeState: the entry points of its SDPA path - MathLM.new_state / prefill / decode_step
    with decode_impl "sdpa" (ultraviolet/model.py:861-872, 880-1008) - on the same kernels."""
    sdpa = kv_dtype in (None, "sdpa")
    if sdpa:
        kv_dtype = "fp16"
    if kv_dtype not in ("int8", "fp16"):
        raise L.UvmiError(f"kv_dtype {kv_dtype!r}: the KV layouts are 'int8' and 'fp16' (unquantized, in the compute dtype)")
    if kv_dtype == "fp16" and dtype not in (torch.float16, torch.bfloat16):
        raise L.UvmiError("an unquantized KV cache needs a 16-bit engine dtype")
    cfg = as_uvconfig(model.cfg)
    sd = model.state_dict()
    dev = device or next(iter(sd.values())).device
    if torch.device(dev).type != "cuda":
        raise L.UvmiError("patch_model needs the model on a GPU (there is no CPU path)")
    eng = UVEngine(UVWeights(cfg, sd, dtype, dev), max_tokens)

    def new_state(self, batch, max_len, dtype=torch.float16, device=None):
        # (an unquantized cache is kept in the engine's activation dtype, whatever the caller's compute dtype is called)
        if sdpa:
            return DecodeState(cfg, batch, max_len, eng.dtype, device or dev)
        return KernelDecodeState(cfg, batch, max_len, eng.dtype if kv_dtype == "fp16" else dtype, device or dev, kv_dtype)

    def decode_step(self, tok, st, g_len=0, skip_attn=False):
        return decode_step_fast(self, tok, st, g_len, skip_attn, num_splits, backend)

    model.__dict__["_uvmi_engine"] = eng
    _remember_stamp(model)
    model.__dict__["new_state"] = types.MethodType(new_state, model)
    model.__dict__["prefill"] = types.MethodType(prefill_fast, model)
    model.__dict__["decode_step"] = types.MethodType(decode_step, model)
    return model


def unpatch_model(model):
    for n in ("new_state", "prefill", "decode_step", "_uvmi_engine", "_uvmi_stamp", "_uvmi_quick", "_uvmi_live"):
        model.__dict__.pop(n, None)
    return model


@torch.no_grad()
def sync_patched_weights(model) -> None:
    """Refresh the engine's fused tensors in place from model.state_dict() (device addresses are kept, so captured graphs
    stay valid).  Called by the patched methods themselves when a parameter's version counter moved; call it by hand
    after replacing parameter storage in a way torch does not version (e.g. through .data of a view)."""
    eng = model.__dict__.get("_uvmi_engine")
    if eng is None:
        raise L.UvmiError("model has not been patched: call patch_model(model) first")
    eng.w.load_(_live_tensors(model))
    _remember_stamp(model)
