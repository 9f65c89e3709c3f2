"""UV-50M forward for inference on the HIP kernels: int8 KV state, one decode step for a ragged batch, packed prefill.

Mirrors ultraviolet/kernels/fast_decode.py of the reference (KernelDecodeState :21-57, decode_step_fast :272-334,
_prefill_packed / prefill_packed_host :117-269) and the layer math of ultraviolet/model.py (Attention.qkv / post
:302-335, Block.finish :567-571, MathLM.logits :824-827).  The GEMMs are torch (hipBLASLt) calls on preallocated
buffers; everything between them is one fused HIP kernel per stage, and K/V go straight into the int8 cache.
One decode step is a fixed launch sequence with no host synchronisation: it reads per-row positions on the device, so
a single captured graph serves every context length (the reference needs one graph per 1024-token bucket,
model.py:1099-1100)."""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch
from torch import Tensor

from .. import _lib as L
from ..kernels.decode_attn import (build_attn_args, build_fused_args, decode_attention, decode_attention_fused, decode_attention_post,
                                   rope_table)
from ..kernels.gemm import RESID, SWIGLU, gemm_tn
from ..kernels.kv_quant import kv_write
from ..kernels.varlen_attn import packed_attention
from ..kernels.fused_sample import fused_sample_seeded, greedy_sample
from .config import UVConfig
from .weights import UVWeights


class KVState:
    """Slot-indexed KV cache (reference: KernelDecodeState, fast_decode.py:21-57): per layer k, v (B, K, S, hd) int8
    and k_scale, v_scale (B, K, S) fp16 with S = max_len on global layers and min(window, max_len) on local (ring)
    layers; pos / starts (B,) int64 on the device.  pos is the next position to write.  kv_dtype "fp16" (the
    reference's name for "unquantized") keeps k, v in `dtype`, the activation type, with no scales."""

    def __init__(self, cfg: UVConfig, B: int, max_len: int, device="cuda", kv_dtype: str = "int8", dtype=torch.bfloat16):
        # Global caches are allocated with S rounded up to 32 slots: the MFMA attention kernel streams 32-key tiles and
        # needs S % 4 == 0 for its 8-byte scale loads (other S fall back to the generic kernel).  Ring length is unchanged.
        self.local_len = min(cfg.window, max_len)
        max_len = (max_len + 31) // 32 * 32
        self.cfg, self.B, self.max_len = cfg, B, max_len
        assert kv_dtype in ("int8", "fp16") and (kv_dtype == "int8" or dtype in (torch.float16, torch.bfloat16))
        self.kv_dtype, self.quantized = kv_dtype, kv_dtype == "int8"
        cdt = torch.int8 if self.quantized else dtype
        dev = torch.device(device)
        self.k, self.v, self.k_scale, self.v_scale = [], [], [], []
        for l in range(cfg.n_layers):
            S = max_len if cfg.is_global(l) else self.local_len
            shp = (B, cfg.n_kv_heads, S, cfg.head_dim)
            self.k.append(torch.zeros(shp, dtype=cdt, device=dev))
            self.v.append(torch.zeros(shp, dtype=cdt, device=dev))
            self.k_scale.append(torch.zeros(shp[:3], dtype=torch.float16, device=dev) if self.quantized else None)
            self.v_scale.append(torch.zeros(shp[:3], dtype=torch.float16, device=dev) if self.quantized else None)
        self.pos = torch.zeros(B, dtype=torch.long, device=dev)
        self.starts = torch.zeros(B, dtype=torch.long, device=dev)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.k + self.v + self.k_scale + self.v_scale if t is not None)

    @torch.no_grad()
    def copy_rows(self, src: Tensor, dst: Tensor, upto: int):
        """Cache rows dst <- cache rows src for the first `upto` slots of every layer, with pos and starts (src, dst: (n,)
        int64 on the device).  A sequence's cache depends only on its own tokens and quantisation is per row, so a prompt
        shared by several sequences is prefilled once and copied: the copies hold the bytes their own prefill would write."""
        for l in range(self.cfg.n_layers):
            for t in (self.k[l], self.v[l], self.k_scale[l], self.v_scale[l]):
                if t is not None:
                    n = min(upto, t.size(2))
                    t[dst, :, :n] = t[src, :, :n]
        self.pos[dst] = self.pos[src]
        self.starts[dst] = self.starts[src]


def kv_bytes_per_seq(cfg: UVConfig, ctx: int) -> int:
    """int8 cache bytes of one sequence at context ctx (reference: fast_decode.py:64-67)."""
    per_pos = 2 * cfg.n_kv_heads * (cfg.head_dim + 2)
    return sum(per_pos * (ctx if cfg.is_global(l) else min(ctx, cfg.window)) for l in range(cfg.n_layers))


def rms_norm_eps(dtype: torch.dtype) -> float:
    """eps that torch.nn.functional.rms_norm(x, eps=None) uses for this dtype in the installed torch (the reference relies
    on that default, model.py:190-191): machine epsilon of the dtype in some releases, of fp32 in others.  Probed once on
    the CPU with a vector small enough that the two candidates give clearly different results."""
    x = torch.full((8,), 2.0 ** -6, dtype=dtype)
    y = float(torch.nn.functional.rms_norm(x, (8,)).float()[0])
    cands = [float(torch.finfo(dtype).eps), float(torch.finfo(torch.float32).eps)]
    refs = [2.0 ** -6 / (2.0 ** -12 + e) ** 0.5 for e in cands]
    return cands[int(np.argmin([abs(y - r) for r in refs]))]


class UVEngine:
    def __init__(self, weights: UVWeights, max_tokens: int, skinny_rows: int = 192, fold_qkv_rows: int = 1 << 30, fold_o_rows: int = 1 << 30,
                 fold_gu_rows: int = 1 << 30, lean: bool = True, fold: bool = True, gemm_config: int = 0,
                 tiled_prefill: bool = True, big_rows: int = 12288, fold_down_rows: tuple = (800, 1632), general_skinny_rows: int = 384):
        """max_tokens: largest number of token rows one forward call processes (decode rows + packed prefill tokens).
        skinny_rows: decode passes of at most this many rows run every projection on the skinny GEMM (general_skinny_rows:
        the same for passes of the general path); fold_qkv_rows, fold_o_rows,
        fold_gu_rows: above skinny_rows, row counts up to which the QKV projection (with the pre-norm), the output
        projection (with the residual update) and the gate-up projection (with the pre-norm and the SwiGLU) run on this
        library's GEMM kernels instead of the vendor library's (see _trunk_folded); lean / fold: the launch plans that drop
        the residual-add and norm launches (off: the general path); gemm_config: form of the hand-written GEMM (0: its own
        choice by size; tests force the tiled forms at a few rows); big_rows: passes of the general path with at least this
        many rows (a packed prefill, a mixed pass) run the down projection too on this library's GEMM, whose 256 x 256 tile
        form is faster than the vendor library there (the other three projections run on it from 448 rows); fold_down_rows:
        (first, last) row count of decode passes whose down projection runs on this library's tiled GEMM.  The defaults are the measured
        optimum on UV-50M."""
        self.w, self.cfg = weights, weights.cfg
        cfg, dt, dev = self.cfg, weights.dtype, weights.device
        assert cfg.head_dim == 64, "the fused kernels are written for head_dim 64"
        self.dtype, self.device, self.max_tokens = dt, dev, max_tokens
        self.dt_code = L.dtype_code(dt)
        self.eps = rms_norm_eps(dt)
        # the attention kernels' query operand: the activation type; an fp32 engine keeps fp32 queries, which run on the plain
        # fp32 attention kernel (no 16-bit rounding of q or of the probabilities anywhere on its path)
        self.q_dtype = dt
        n, d, H, K, hd, f = max_tokens, cfg.d_model, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, cfg.d_ff
        e = lambda *s, dtype=dt: torch.empty(*s, dtype=dtype, device=dev)
        self.buf = dict(x=e(n, d), xn=e(n, d), h=e(n, d), qkv=e(n, (H + 2 * K) * hd), q=e(n, H, hd, dtype=self.q_dtype),
                        k=e(n, K, hd), v=e(n, K, hd), zg=e(n, H * hd), a=e(n, d), gu=e(n, 2 * f), act=e(n, f), m=e(n, d),
                        vhat=e(n, K, hd, dtype=torch.float32), gate=e(n, H, dtype=torch.float32))
        # decode steps of a 16-bit engine take q, k, v and the gate logits from one extended projection and leave the
        # post-processing to the attention kernel (one launch less per layer)
        self.fuse_qkv = dt in (torch.bfloat16, torch.float16) and cfg.n_heads // cfg.n_kv_heads <= 8 and cfg.n_pairs in (0, 16)
        self.qkvx_keep = None
        # Passes of at most this many rows run every projection on the skinny GEMM (the down projection with the block's
        # second residual update in its epilogue); above it the folded plan (tiled GEMMs, the vendor library for the down
        # projection).  Measured on UV-50M decode steps inside a rollout: 0.369 against 0.388 ms at 192 rows, 0.424 against
        # 0.415 at 256, 0.466 against 0.460 at 320, equal at 384.
        self.skinny_rows = int(skinny_rows) if dt in (torch.bfloat16, torch.float16) else 0
        # passes of the general path (prefill, mixed steps, layers without the fused attention) keep the skinny GEMM up to
        # this many rows: their alternative below 448 rows is the vendor library with separate SwiGLU and norm launches
        self.general_skinny_rows = int(general_skinny_rows) if dt in (torch.bfloat16, torch.float16) else 0
        # above skinny_rows the skinny kernel still carries the QKV projection (with the pre-norm) and the output projection
        # (with the residual update) up to these many rows
        self.fold_qkv_rows = int(fold_qkv_rows)
        self.fold_o_rows, self.fold_gu_rows = int(fold_o_rows), int(fold_gu_rows)
        self.lean, self.fold, self.gemm_config = bool(lean), bool(fold), int(gemm_config)
        self.tiled_prefill = bool(tiled_prefill)
        self.big_rows = int(big_rows)
        # the folded plan's down projection runs on this library's tiled GEMM between these row counts (measured inside the
        # decode step: 4 - 11 us per step faster than the vendor library's there, slower below and above)
        self.fold_down_rows = (int(fold_down_rows[0]), int(fold_down_rows[1]))
        self.head_own_rows = 288       # decode steps of at most this many rows run the head GEMM on this library's kernel (own_head_ok)
        self.hidden_is_raw = False
        self._rope_tabs: dict[int, Tensor] = {}  # rotation tables by position count, kept for the engine's life (graphs hold them)
        if self.fuse_qkv:
            self.buf["qkvx"] = e(n, UVWeights.qkv_ext_rows(cfg))
        self.pf_ws = torch.empty(L.lib().uvmi_prefill_attn_workspace_bytes(n), dtype=torch.uint8, device=dev)  # fails now if the library is missing

    # ------------------------------------------------------------------------------------------------ kernels
    def _embed_norm(self, tok: Tensor, n: int):
        b = self.buf
        rc = L.lib().uvmi_embed_norm(self.w.embed.data_ptr(), self.dt_code, self.cfg.vocab_size, tok.data_ptr(), n,
                                     self.cfg.d_model, self.eps, b["x"].data_ptr(), b["xn"].data_ptr(), L.stream_ptr(tok))
        L.check(rc, "uvmi_embed_norm")

    def _add_norm(self, x: Tensor, y: Tensor, a: float, bb: float, n: int, h_out: Tensor | None, n_out: Tensor):
        rc = L.lib().uvmi_add_norm(x.data_ptr(), y.data_ptr(), self.dt_code, a, bb, n, self.cfg.d_model, self.eps,
                                   None if h_out is None else h_out.data_ptr(), n_out.data_ptr(), L.stream_ptr(x))
        L.check(rc, "uvmi_add_norm")

    def _qkv_post(self, l: int, tok: Tensor, pos: Tensor, rows: Tensor | None, last_pos: Tensor | None, st: KVState | None,
                  n: int, write_cache: bool = True, ext: bool = False):
        """ext: the rows come from the extended projection (buf qkvx), whose last columns are the gates' logits: the
        normalised block input is then not read."""
        cfg, b, W = self.cfg, self.buf, self.w.layers[l]
        glob = cfg.is_global(l)
        a = L.QkvPostArgs()
        a.qkv, a.dtype, a.xn = b["qkvx" if ext else "qkv"].data_ptr(), self.dt_code, b["xn"].data_ptr()
        if ext:
            a.qkv_ld, a.ext_logits = b["qkvx"].stride(0), 1
        has_ve = cfg.has_ve(l)
        if has_ve:
            a.ve_table, a.ve_gate, a.tok = self.w.value_embed.data_ptr(), W["ve_gate"].data_ptr(), tok.data_ptr()
        a.pos = pos.data_ptr()
        a.rows = None if rows is None else rows.data_ptr()
        a.last_pos = None if last_pos is None else last_pos.data_ptr()
        a.inv_freq = self.w.inv_freq.data_ptr()
        a.q_out, a.q_dtype = b["q"].data_ptr(), L.dtype_code(self.q_dtype)
        a.k_out, a.v_out = b["k"].data_ptr(), b["v"].data_ptr()
        if st is not None and write_cache and st.quantized:
            kc, ks = st.k[l], st.k_scale[l]
            a.k_cache, a.v_cache, a.k_scale, a.v_scale = kc.data_ptr(), st.v[l].data_ptr(), ks.data_ptr(), st.v_scale[l].data_ptr()
            a.scb, a.sch, a.scs, a.ssb, a.ssh = kc.stride(0), kc.stride(1), kc.stride(2), ks.stride(0), ks.stride(1)
            a.S = kc.size(2)
        a.n, a.vocab = n, cfg.vocab_size
        a.H, a.KH, a.hd, a.d, a.ve_ch, a.n_pairs = cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, cfg.d_model, cfg.ve_gate_channels, cfg.n_pairs
        a.ring, a.has_ve = int(not glob), int(has_ve)
        a.rope = int(((not glob) or cfg.global_rope) and cfg.n_pairs > 0)
        if a.rope and st is not None:   # cos / sin from the table of the state's positions instead of per-token cosf / sinf
            tab = self.rope_table(st.max_len)
            a.rope_table, a.rope_positions = tab.data_ptr(), tab.size(0)
        a.eps = self.eps
        if cfg.xsa:
            a.vhat_out, a.xsa_eps = b["vhat"].data_ptr(), float(cfg.xsa_eps)
        if W["attn_gate"] is not None:
            a.gate_w, a.gate_ch, a.gate_out = W["attn_gate"].data_ptr(), cfg.gate_ch, b["gate"].data_ptr()
        L.check(L.lib().uvmi_qkv_post(C.byref(a), L.stream_ptr(pos)), "uvmi_qkv_post")
        if st is not None and write_cache and not st.quantized:
            self._write_kv16(l, pos, rows, last_pos, st, n)

    def _write_kv16(self, l: int, pos: Tensor, rows: Tensor | None, last_pos: Tensor | None, st: KVState, n: int):
        """Unquantized caches: buf k / v of the n rows go to slot pos (pos % S on a ring) of their cache rows - the two
        kv_write calls of the reference's step (fast_decode.py:291-294, 315-317).  Dropped, as the int8 append drops them:
        padding rows, positions past a linear cache, and prompt positions a ring will not keep (older than last_pos - S)."""
        cfg, b = self.cfg, self.buf
        K = cfg.n_kv_heads
        S = st.k[l].size(2)
        ring = not cfg.is_global(l)
        row = torch.arange(n, device=pos.device) if rows is None else rows[:n]
        p = pos[:n]
        slot = torch.remainder(p, S) if ring else p
        ok = (row >= 0) & (p >= 0) & (slot < S)
        if ring and last_pos is not None:
            ok &= p > last_pos[:n] - S
        flat = (row[:, None] * K + torch.arange(K, device=pos.device)[None, :]) * S + slot[:, None]
        flat = torch.where(ok[:, None], flat, torch.full_like(flat, -1)).reshape(-1).contiguous()
        kv_write(st.k[l], None, flat, b["k"][:n])
        kv_write(st.v[l], None, flat, b["v"][:n])

    def _attn_post(self, l: int, z: Tensor, n: int, off: int = 0):
        """XSA + gate of rows off..off+n of the call (z holds just those rows); writes buf zg[off:off+n]."""
        cfg, b, W = self.cfg, self.buf, self.w.layers[l]
        rc = L.lib().uvmi_attn_post(z.data_ptr(), L.dtype_code(z.dtype), b["v"][off:].data_ptr(), b["xn"][off:].data_ptr(), self.dt_code,
                                    None if W["attn_gate"] is None else W["attn_gate"].data_ptr(),
                                    None if W["xsa"] is None else W["xsa"].data_ptr(), float(cfg.xsa_eps), n, cfg.n_heads,
                                    cfg.n_kv_heads, cfg.head_dim, cfg.d_model, cfg.gate_ch, b["zg"][off:].data_ptr(), L.stream_ptr(z))
        L.check(rc, "uvmi_attn_post")

    def _swiglu(self, n: int):
        b = self.buf
        rc = L.lib().uvmi_swiglu(b["gu"].data_ptr(), self.dt_code, n, self.cfg.d_ff, b["act"].data_ptr(), L.stream_ptr(b["gu"]))
        L.check(rc, "uvmi_swiglu")

    def _swiglu_norm(self, h: Tensor, n: int):
        """buf act = SwiGLU of rmsnorm(h) @ gu.T, from buf gu = h @ gu.T (the norm as a row scale of the product)."""
        b = self.buf
        rc = L.lib().uvmi_swiglu_norm(b["gu"].data_ptr(), h.data_ptr(), self.dt_code, n, self.cfg.d_ff, self.cfg.d_model, self.eps,
                                      b["act"].data_ptr(), L.stream_ptr(h))
        L.check(rc, "uvmi_swiglu_norm")

    # ------------------------------------------------------------------------------------------------ trunk
    def cache_attention(self, l: int, q: Tensor, st: KVState, pos: Tensor, starts: Tensor, n: int, rows: Tensor | None = None,
                        off: int = 0):
        """Decode attention of layer l over the cache (int8, or unquantized) with the fused XSA + gate epilogue for the n rows that sit at
        off..off+n of the call's buffers (q is already that slice); writes buf zg[off:off+n] and returns None, or, where
        the fused epilogue does not apply, returns the plain attention output for _attn_post."""
        cfg, b, W = self.cfg, self.buf, self.w.layers[l]
        glob = cfg.is_global(l)
        S = st.k[l].size(2)
        kw = dict(window=0 if glob else cfg.window, ring=not glob, k_scale=st.k_scale[l], v_scale=st.v_scale[l], rows=rows)
        # the MFMA kernel (which carries the epilogue) streams 32-key tiles: rings need S % 32 == 0, linear int8 caches
        # S % 4 == 0; it serves int8 caches and caches in the q dtype
        mfma_cache = q.dtype != torch.float32 and (st.quantized or (st.k[l].dtype == q.dtype and q.dtype in (torch.float16, torch.bfloat16)))
        if mfma_cache and cfg.xsa and cfg.n_heads // cfg.n_kv_heads <= 8 and S % (4 if glob else 32) == 0 and S >= 32:
            out = b["zg"][off:off + n].view(n, cfg.n_heads, cfg.head_dim)
            decode_attention_post(q, st.k[l], st.v[l], pos, starts, cfg.attn_scale, vhat=b["vhat"][off:off + n],
                                  gate=None if W["attn_gate"] is None else b["gate"][off:off + n], xsa=W["xsa"], out=out, **kw)
            return None
        return decode_attention(q, st.k[l], st.v[l], pos, starts, cfg.attn_scale, num_splits=1, **kw)

    def prompt_attention(self, l: int, q: Tensor, N: int, cu: Tensor):
        """Causal (windowed on local layers) attention of the N packed prompt tokens at the head of the call's buffers over
        their own unquantized K / V (buf k, v).  Where the MFMA kernel runs (16-bit engine) XSA and the gate ride in its
        epilogue - it writes buf zg[:N] and None is returned; otherwise the plain attention output is returned for
        _attn_post.  The segment table of cu is built by layer 0's call and reused by the other layers of the pass."""
        cfg, b, W = self.cfg, self.buf, self.w.layers[l]
        w = 0 if cfg.is_global(l) else cfg.window
        kw = dict(workspace=self.pf_ws, segments_ready=l > 0)
        if (cfg.xsa and self.dtype in (torch.bfloat16, torch.float16) and self.q_dtype == self.dtype and cfg.head_dim == 64
                and cfg.n_heads // cfg.n_kv_heads <= 8):
            out = b["zg"][:N].view(N, cfg.n_heads, cfg.head_dim)
            packed_attention(q, b["k"][:N], b["v"][:N], cu, cfg.attn_scale, w, out=out,
                             post=(b["vhat"][:N], None if W["attn_gate"] is None else b["gate"][:N], W["xsa"]), **kw)
            return None
        return packed_attention(q, b["k"][:N], b["v"][:N], cu, cfg.attn_scale, w, **kw)

    def fused_layer_ok(self, l: int, st: KVState) -> bool:
        """Whether layer l's decode attention can take the fused path: the MFMA kernel streams 32-key tiles."""
        S = st.k[l].size(2)
        return self.fuse_qkv and (st.quantized or st.k[l].dtype == self.dtype) and S % 32 == 0 and S >= 32

    def rope_table(self, n_positions: int) -> Tensor:
        """cos / sin of every position below n_positions in the activation type's rounding, built once per size."""
        t = self._rope_tabs.get(n_positions)
        if t is None:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("the rotation table must exist before a graph is captured: call rope_table(state.max_len) first")
            t = self._rope_tabs[n_positions] = rope_table(self.w.inv_freq, n_positions, self.dtype)
        return t

    def _fuse_dict(self, l: int, tok: Tensor, st: KVState) -> dict:
        cfg = self.cfg
        glob = cfg.is_global(l)
        has_ve = cfg.has_ve(l)
        rope = ((not glob) or cfg.global_rope) and cfg.n_pairs > 0
        return dict(ext_col=(cfg.n_heads + 2 * cfg.n_kv_heads) * cfg.head_dim, has_gate=cfg.gate_ch > 0, tok=tok if has_ve else None,
                    ve_table=self.w.value_embed if has_ve else None, vocab=cfg.vocab_size, rope_table=self.rope_table(st.max_len) if rope else None,
                    n_pairs=cfg.n_pairs, rope=rope, eps=self.eps, xsa_eps=cfg.xsa_eps)

    def fused_cache_attention(self, l: int, tok: Tensor, st: KVState, pos: Tensor, starts: Tensor, n: int, rows: Tensor | None = None):
        """Decode attention of layer l straight from buf qkvx (the extended projection of the n rows): QK-norm, rotation,
        value embedding, int8 append, attention over lo..pos, XSA and gate in one launch; writes buf zg."""
        cfg, b, W = self.cfg, self.buf, self.w.layers[l]
        glob = cfg.is_global(l)
        out = b["zg"][:n].view(n, cfg.n_heads, cfg.head_dim)
        decode_attention_fused(b["qkvx"][:n], cfg.n_heads, st.k[l], st.v[l], pos, starts, cfg.attn_scale, window=0 if glob else cfg.window,
                               ring=not glob, k_scale=st.k_scale[l], v_scale=st.v_scale[l], xsa=W["xsa"], out=out,
                               fuse=self._fuse_dict(l, tok, st), rows=rows)

    def fused_attention_args(self, l: int, qkvx: Tensor, tok: Tensor, st: KVState, pos: Tensor, starts: Tensor, n: int,
                             rows: Tensor | None = None):
        """The uvmi_attn_args struct fused_cache_attention launches for layer l, on a given copy of that layer's extended
        projection (qkvx_keep): lets a benchmark re-issue exactly the step's launches through the C ABI.  Re-issuing it
        on the step's own positions rewrites the same K/V bytes."""
        cfg, b, W = self.cfg, self.buf, self.w.layers[l]
        glob = cfg.is_global(l)
        out = b["zg"][:n].view(n, cfg.n_heads, cfg.head_dim)
        return build_fused_args(qkvx[:n], cfg.n_heads, st.k[l], st.v[l], pos, starts, cfg.attn_scale, 0 if glob else cfg.window, not glob,
                                st.k_scale[l], st.v_scale[l], W["xsa"], out, self._fuse_dict(l, tok, st), rows)

    def cache_attention_args(self, l: int, st: KVState, pos: Tensor, starts: Tensor, n: int, rows: Tensor | None = None):
        """The uvmi_attn_args struct cache_attention would launch for layer l on the engine's buffers (fused path only):
        lets a benchmark re-issue exactly the step's attention launches through the C ABI without the Python wrapper."""
        cfg, b, W = self.cfg, self.buf, self.w.layers[l]
        glob = cfg.is_global(l)
        out = b["zg"][:n].view(n, cfg.n_heads, cfg.head_dim)
        return build_attn_args(b["q"][:n], st.k[l], st.v[l], pos, starts, cfg.attn_scale, 0 if glob else cfg.window, not glob,
                               st.k_scale[l], st.v_scale[l], 1, out, 0, rows,
                               (b["vhat"][:n], None if W["attn_gate"] is None else b["gate"][:n], W["xsa"], out.dtype))

    def _trunk(self, tok: Tensor, pos: Tensor, n: int, attn, rows=None, last_pos=None, st: KVState | None = None,
               fused_attn=None, defer_final_norm: bool = False) -> Tensor:
        """n token rows through all layers; attn(l, q (n, H, hd)) -> z (n, H, hd) (or None when it wrote the post-processed
        result to buf zg itself) runs after K/V of the layer have been appended to the cache and written unquantized to
        buf k / v.  Returns the final normed hidden (n, d) (a buffer).  defer_final_norm: a plan whose last block leaves the
        hidden un-normalised returns it as it is and sets self.hidden_is_raw - the caller's head GEMM then carries the final
        norm as the row scale of its product (head_of), and the norm launch goes away."""
        cfg, b = self.cfg, self.buf
        assert n <= self.max_tokens
        self._embed_norm(tok, n)
        x, xn = b["x"][:n], b["xn"][:n]
        skinny_rows = self.skinny_rows if fused_attn is not None else max(self.skinny_rows, self.general_skinny_rows)
        skinny = n <= skinny_rows and cfg.d_model % 64 == 0 and cfg.d_model <= 960 and (cfg.n_heads * cfg.head_dim) % 64 == 0
        mm = (lambda a, w, out: gemm_tn(a, w, out)) if skinny else (lambda a, w, out: torch.mm(a, w.t(), out=out))
        # Small passes whose every layer takes the fused attention never need the normalised hidden in memory: the block's
        # second residual update then rides on the down projection and the next block's pre-norm on its QKV projection (a row
        # scale of the product), and only the final norm is a launch of its own.
        lean = (skinny and fused_attn is not None and self.lean
                and all("gu_il" in W and self.fused_layer_ok(l, st) for l, W in enumerate(self.w.layers))
                and cfg.d_ff % 64 == 0 and cfg.d_ff <= 1984)
        # Larger passes under the same condition keep the library GEMMs but still never add a launch for a residual update or
        # for the MLP's pre-norm: both residual updates are the library's own C = alpha A B + beta C on the hidden in place,
        # and the pre-norm is a row scale inside the SwiGLU launch (7 launches per layer where the general path has 8; 6 while
        # the QKV projection with the pre-norm in it is still faster on the skinny kernel).
        folded = (not skinny and fused_attn is not None and self.fold and self.dtype != torch.float32
                  and all(self.fused_layer_ok(l, st) for l in range(cfg.n_layers)) and cfg.d_ff % 8 == 0)
        self.hidden_is_raw = False
        if folded:
            return self._trunk_folded(n, fused_attn, defer_final_norm)
        fold_mlp = not skinny and self.dtype != torch.float32 and cfg.d_ff % 8 == 0 and self.fold
        tiled_gu = (fold_mlp and self.tiled_prefill and n >= 448 and cfg.d_model % 64 == 0
                    and all("gu_il" in W for W in self.w.layers))
        # Passes of the general path with many rows (a packed prefill, a mixed step): the QKV and output projections run on this
        # library's GEMM (64 x 64 / 128 x 128 tiles, 256 x 256 from big_rows rows on - faster than the vendor library's at these
        # shapes), the output projection with the residual update in place; from big_rows rows on the down projection too.
        own = (fold_mlp and tiled_gu and (cfg.n_heads * cfg.head_dim) % 64 == 0 and cfg.d_ff % 64 == 0 and cfg.d_model % 8 == 0)
        own_down = own and n >= self.big_rows
        if own:
            mm = lambda a, w, out: gemm_tn(a, w, out, config=self.gemm_config)
        # ... and with the extended projection (q, k, v and the gates' logits) the block's pre-norm rides on the QKV GEMM as a
        # row scale and the post-processing reads the logits from the projection: the normalised hidden is not written between
        # blocks (it is formed on demand for a layer whose attention leaves its epilogue to _attn_post)
        own_ext = own and self.fuse_qkv and fused_attn is None and all("wqkv_ext" in W for W in self.w.layers)
        x_is_normed = True   # buf xn holds rmsnorm(x)
        for l, W in enumerate(self.w.layers):
            if fused_attn is not None and self.fused_layer_ok(l, st):
                # decode rows of a 16-bit engine: the projection also forms the gate logits, and fused_attn(l) does the
                # post-processing, the cache append, the attention and its epilogue in one launch (writes buf zg)
                if x_is_normed:
                    mm(xn, W["wqkv_ext"], b["qkvx"][:n])
                else:
                    gemm_tn(x, W["wqkv_ext"], b["qkvx"][:n], norm_eps=self.eps)
                if self.qkvx_keep is not None:   # a benchmark re-issues this layer's launch later on the same projection
                    self.qkvx_keep[l][:n].copy_(b["qkvx"][:n])
                fused_attn(l)
            elif own_ext:
                if x_is_normed:
                    gemm_tn(xn, W["wqkv_ext"], b["qkvx"][:n], config=self.gemm_config)
                else:
                    gemm_tn(x, W["wqkv_ext"], b["qkvx"][:n], norm_eps=self.eps, config=self.gemm_config)
                self._qkv_post(l, tok, pos, rows, last_pos, st, n, ext=True)
                z = attn(l, b["q"][:n])
                if z is not None:
                    if not x_is_normed:
                        self._add_norm(x, x, 1.0, 0.0, n, None, b["xn"])
                        x_is_normed = True
                    self._attn_post(l, z, n)
            else:
                mm(xn, W["wqkv"], b["qkv"][:n])
                self._qkv_post(l, tok, pos, rows, last_pos, st, n)
                z = attn(l, b["q"][:n])
                if z is not None:   # None: the attention kernel already applied XSA + gate and wrote buf zg
                    self._attn_post(l, z, n)
            if skinny and "gu_il" in W:
                # the residual update rides on the output projection (h = resid_attn * x + post_attn * a) and the MLP's
                # pre-norm on the gate-up projection (a row scale of the product), whose epilogue is the SwiGLU: two
                # launches where the general path has five
                gemm_tn(b["zg"][:n], W["wo"], b["h"][:n], epilogue=RESID, resid=x, ca=W["resid_attn"], cb=W["post_attn"])
                gemm_tn(b["h"][:n], W["gu_il"], b["act"][:n], epilogue=SWIGLU, norm_eps=self.eps)
            elif fold_mlp:
                # 16-bit passes of any size and attention path: both residual updates are the library's C = alpha A B + beta C
                # on the hidden in place and the MLP's pre-norm is the row scale inside the SwiGLU launch; the block ends
                # with the norm the next block's projection and post-processing read
                if own:
                    gemm_tn(b["zg"][:n], W["wo"], x, epilogue=RESID, resid=x, ca=W["resid_attn"], cb=W["post_attn"], config=self.gemm_config)
                else:
                    torch.addmm(x, b["zg"][:n], W["wo"].t(), beta=W["resid_attn"], alpha=W["post_attn"], out=x)
                if tiled_gu:   # the tiled GEMM with the pre-norm and the SwiGLU in it: the (n, 2 f) product is never written
                    gemm_tn(x, W["gu_il"], b["act"][:n], epilogue=SWIGLU, norm_eps=self.eps, config=self.gemm_config)
                else:
                    torch.mm(x, W["gu"].t(), out=b["gu"][:n])
                    self._swiglu_norm(x, n)
                if own_down:
                    gemm_tn(b["act"][:n], W["down"], x, epilogue=RESID, resid=x, ca=W["resid_mlp"], cb=W["post_mlp"], config=self.gemm_config)
                else:
                    torch.addmm(x, b["act"][:n], W["down"].t(), beta=W["resid_mlp"], alpha=W["post_mlp"], out=x)
                if own_ext:
                    x_is_normed = False
                else:
                    self._add_norm(x, x, 1.0, 0.0, n, None, b["xn"])
                continue
            else:
                mm(b["zg"][:n], W["wo"], b["a"][:n])
                # h = resid_attn * x + post_attn * a ; n = rmsnorm(h)
                self._add_norm(x, b["a"][:n], W["resid_attn"], W["post_attn"], n, b["h"], b["xn"])
                mm(xn, W["gu"], b["gu"][:n])
                self._swiglu(n)
            if lean:
                # x = resid_mlp * h + post_mlp * m in the down projection's epilogue (in place of the residual-add + norm launch)
                gemm_tn(b["act"][:n], W["down"], x, epilogue=RESID, resid=b["h"][:n], ca=W["resid_mlp"], cb=W["post_mlp"])
                x_is_normed = False
            else:
                torch.mm(b["act"][:n], W["down"].t(), out=b["m"][:n])   # (K = d_ff: 26 K-steps per strip, the library is faster)
                # x = resid_mlp * h + post_mlp * m ; xn = rmsnorm(x) (next block's pre-norm, or the final norm)
                self._add_norm(b["h"][:n], b["m"][:n], W["resid_mlp"], W["post_mlp"], n, b["x"], b["xn"])
        if not x_is_normed:
            if defer_final_norm and self.own_head_ok(n):
                self.hidden_is_raw = True
                return x
            self._add_norm(x, x, 1.0, 0.0, n, None, b["xn"])   # the final norm
        return xn

    def _trunk_folded(self, n: int, fused_attn, defer_final_norm: bool = False) -> Tensor:
        """The layers of _trunk for a pass of many rows whose every layer takes the fused attention; buf x and xn hold the
        embedded rows and their norm on entry.  Five launches per layer: QKV projection with the block's pre-norm as a row
        scale, fused attention, output projection with the residual update in place, gate-up projection with the MLP's
        pre-norm and the SwiGLU in its epilogue (the tiled GEMM of this library: the (n, 2 f) intermediate and the
        normalised hidden are never written), down projection with the residual update (the vendor library's
        C = alpha A B + beta C: at K = d_ff it is still the faster kernel)."""
        cfg, b = self.cfg, self.buf
        x, xn = b["x"][:n], b["xn"][:n]
        gc = self.gemm_config
        sk_ok = cfg.d_model % 64 == 0 and (cfg.n_heads * cfg.head_dim) % 64 == 0
        sk_qkv, sk_o = sk_ok and n <= self.fold_qkv_rows, sk_ok and n <= self.fold_o_rows
        for l, W in enumerate(self.w.layers):
            if l == 0:      # (the embedding's norm exists already: the same product as on the general path, bit for bit -
                            # the tiled GEMM of this library from 448 rows, where the general path takes it too)
                if sk_qkv and n >= 448:
                    gemm_tn(xn, W["wqkv_ext"], b["qkvx"][:n], config=gc)
                else:
                    torch.mm(xn, W["wqkv_ext"].t(), out=b["qkvx"][:n])
            elif sk_qkv:
                gemm_tn(x, W["wqkv_ext"], b["qkvx"][:n], norm_eps=self.eps, config=gc)
            else:
                self._add_norm(x, x, 1.0, 0.0, n, None, b["xn"])
                torch.mm(xn, W["wqkv_ext"].t(), out=b["qkvx"][:n])
            if self.qkvx_keep is not None:
                self.qkvx_keep[l][:n].copy_(b["qkvx"][:n])
            fused_attn(l)
            # x <- resid_attn * x + post_attn * (zg @ wo.T), in place (every element is read and written by the same lane)
            if sk_o:
                gemm_tn(b["zg"][:n], W["wo"], x, epilogue=RESID, resid=x, ca=W["resid_attn"], cb=W["post_attn"], config=gc)
            else:
                torch.addmm(x, b["zg"][:n], W["wo"].t(), beta=W["resid_attn"], alpha=W["post_attn"], out=x)
            if sk_ok and "gu_il" in W and n <= self.fold_gu_rows:
                gemm_tn(x, W["gu_il"], b["act"][:n], epilogue=SWIGLU, norm_eps=self.eps, config=gc)
            else:
                torch.mm(x, W["gu"].t(), out=b["gu"][:n])
                self._swiglu_norm(x, n)
            # x <- resid_mlp * x + post_mlp * (act @ down.T)
            if sk_ok and self.fold_down_rows[0] <= n <= self.fold_down_rows[1] and cfg.d_ff % 64 == 0:
                gemm_tn(b["act"][:n], W["down"], x, epilogue=RESID, resid=x, ca=W["resid_mlp"], cb=W["post_mlp"], config=gc)
            else:
                torch.addmm(x, b["act"][:n], W["down"].t(), beta=W["resid_mlp"], alpha=W["post_mlp"], out=x)
        if defer_final_norm and self.own_head_ok(n):
            self.hidden_is_raw = True
            return x
        self._add_norm(x, x, 1.0, 0.0, n, None, b["xn"])   # the final norm
        return xn

    def own_head_ok(self, n: int) -> bool:
        """Whether head_of runs the head GEMM of n rows on this library's kernel with the final norm in it: 16-bit engines up
        to head_own_rows rows.  Measured on UV-50M (32 768 x 640 head) as the time of a whole graph-replayed decode step
        against the vendor library's GEMM behind a norm launch: 0.3325 against 0.3338 ms at 192 rows, 0.3644 against 0.3699
        at 256, but 0.4137 against 0.4111 at 320 and 0.4363 against 0.4297 at 384 - so the switch sits at 288 rows.  (Alone,
        on cold weights, the kernel takes 11.5 - 25 us at 32 - 384 rows where the vendor library's takes 10 - 22 us plus ~6 us
        of norm launch; at 2048 rows 105 against 87 us.)"""
        cfg = self.cfg
        return (self.dtype in (torch.bfloat16, torch.float16) and n <= self.head_own_rows and cfg.d_model % 64 == 0
                and cfg.d_model >= 128 and cfg.vocab_size % 16 == 0)

    def head_of(self, hidden: Tensor) -> Tensor:
        """head() of what _trunk(defer_final_norm=True) returned: a raw hidden goes through this library's GEMM with the
        final norm as the row scale of the product (128 x 128 tiles; 256 x 256 where they fill the device in whole
        rounds), a normalised one through head()."""
        if not self.hidden_is_raw:
            return self.head(hidden)
        n = hidden.size(0)
        blocks = -(-n // 256)
        config = 5 if n > 384 and blocks % 2 == 0 else 6
        return gemm_tn(hidden, self.w.embed, norm_eps=self.eps, config=config)

    def head(self, hidden: Tensor) -> Tensor:
        """Raw tied-head output (n, V) in the activation dtype: the GEMM MathLM.logits runs before .float() and the
        softcap (model.py:824-827); the sampler applies the softcap."""
        return torch.mm(hidden, self.w.embed.t())

    def logits(self, hidden: Tensor) -> Tensor:
        a, bb, c = self.cfg.softcap
        return a * torch.sigmoid((self.head(hidden).float() + bb) / c)

    # ------------------------------------------------------------------------------------------------ decode
    @torch.no_grad()
    def decode_step(self, tok: Tensor, st: KVState, num_splits: dict | None = None, fuse: bool = True) -> Tensor:
        """One token for all B rows at per-row st.pos (reference: decode_step_fast, fast_decode.py:272-334): append K/V
        at pos first, attend lo..pos, then st.pos += 1.  Returns the final normed hidden (B, d)."""
        cfg = self.cfg
        B = tok.numel()
        pos, starts = st.pos, st.starts
        ns = num_splits or {}

        def attn(l, q):
            key = "global" if cfg.is_global(l) else "local"
            if ns.get(key) in (None, 1):
                return self.cache_attention(l, q, st, pos, starts, B)
            glob = cfg.is_global(l)
            return decode_attention(q, st.k[l], st.v[l], pos, starts, cfg.attn_scale, window=0 if glob else cfg.window, ring=not glob,
                                    k_scale=st.k_scale[l], v_scale=st.v_scale[l], num_splits=ns[key])

        fused = None
        if self.fuse_qkv and not num_splits and fuse:
            fused = lambda l: self.fused_cache_attention(l, tok, st, pos, starts, B)
        h = self._trunk(tok, pos, B, attn, st=st, fused_attn=fused)
        st.pos.add_(1)
        return h

    # ------------------------------------------------------------------------------------------------ prefill
    def pack_prompts(self, prompts: list[list[int]], rows: list[int], max_len: int, left_pad: bool = True) -> dict:
        """Host-built packed indices of a prefill call (reference: prefill_packed_host, fast_decode.py:210-269): per packed
        token its id, position, cache row and the last position of its prompt; cu_seqlens; the packed index of every
        prompt's last token; per prompt the cache row, start and end position.  All as device tensors."""
        dev = self.device
        lens = np.fromiter((len(p) for p in prompts), dtype=np.int64, count=len(prompts))
        assert lens.min() > 0
        T = int(lens.max())
        assert T <= max_len
        starts = (T - lens) if left_pad else np.zeros_like(lens)
        cu = np.zeros(len(prompts) + 1, dtype=np.int64)
        cu[1:] = np.cumsum(lens)
        N = int(cu[-1])
        assert N <= self.max_tokens, f"{N} prefill tokens exceed the engine's max_tokens {self.max_tokens}"
        x = np.concatenate([np.asarray(p, dtype=np.int64) for p in prompts])   # (prompts may be lists or int arrays)
        seg = np.repeat(np.arange(len(prompts), dtype=np.int64), lens)
        pos = np.arange(N, dtype=np.int64) - cu[:-1][seg] + starts[seg]
        rows_np = np.asarray(rows, dtype=np.int64)
        # one host -> device copy for all nine arrays
        parts = [x, pos, rows_np[seg], (starts + lens - 1)[seg], cu, cu[1:] - 1, rows_np, starts, starts + lens]
        flat = torch.from_numpy(np.concatenate(parts)).to(dev)
        tok, pos_t, row, last, cu_t, last_idx, rows_t, starts_t, ends = flat.split([len(a) for a in parts])
        return dict(N=N, tok=tok, pos=pos_t, row=row, last=last, cu=cu_t, last_idx=last_idx, rows=rows_t, starts=starts_t, ends=ends)

    @staticmethod
    def bind_prompts(pk: dict, st: KVState):
        """Point the cache rows of a packed prefill at their prompts: starts = first position, pos = next position."""
        st.starts[pk["rows"]] = pk["starts"]
        st.pos[pk["rows"]] = pk["ends"]

    @torch.no_grad()
    def mixed_step(self, pk: dict, tok_d: Tensor, pos_d: Tensor, starts_d: Tensor, rows_d: Tensor, st: KVState) -> tuple[Tensor, Tensor]:
        """One forward pass over a mixed batch: the packed prompts of `pk` (prefilled into their cache rows) followed by
        n_d decode rows (token tok_d at position pos_d of cache row rows_d; rows_d < 0 marks padding).  Every GEMM, norm
        and the fused QKV post-processing / cache append run once over all N_p + n_d token rows; attention runs as one
        packed causal launch over the prompt tokens and one cache launch over the decode rows per layer.  The reference
        runs these as two passes (its refill prefill, then the decode step: model.py:1296-1313, 1321-1330).
        Returns the final normed hidden of each prompt's last token and of each decode row.  Does not advance st.pos of
        the decode rows (the caller's slot table does), but binds the prompts' rows."""
        Np, nd = pk["N"], tok_d.numel()
        tok, pos = torch.cat([pk["tok"], tok_d]), torch.cat([pk["pos"], pos_d])
        rows, last = torch.cat([pk["row"], rows_d]), torch.cat([pk["last"], pos_d])
        h = self.mixed_trunk(tok, pos, rows, last, Np, nd, pk["cu"], starts_d, st)
        self.bind_prompts(pk, st)
        return h.index_select(0, pk["last_idx"]), h[Np:Np + nd]

    def mixed_trunk(self, tok: Tensor, pos: Tensor, rows: Tensor, last: Tensor, Np: int, nd: int, cu: Tensor, starts_d: Tensor,
                    st: KVState) -> Tensor:
        """The pass of mixed_step over already concatenated per-token arrays (Np packed prompt tokens, then nd decode rows;
        cu: the prompts' cu_seqlens on the device).  Allocation-free apart from the packed attention output, so a caller
        that builds the arrays on the device can capture it in a graph.  Returns the final normed hidden (Np + nd, d)."""
        cfg, b = self.cfg, self.buf
        N = Np + nd
        assert N <= self.max_tokens, f"{N} token rows exceed the engine's max_tokens {self.max_tokens}"
        pos_d, rows_d = pos[Np:N], rows[Np:N]

        def attn(l, q):
            zp = self.prompt_attention(l, q[:Np], Np, cu)
            if zp is not None:
                self._attn_post(l, zp, Np)
            zd = self.cache_attention(l, q[Np:N], st, pos_d, starts_d, nd, rows=rows_d, off=Np)
            if zd is not None:
                self._attn_post(l, zd, nd, off=Np)
            return None

        return self._trunk(tok[:N], pos[:N], N, attn, rows=rows[:N], last_pos=last[:N], st=st)

    @torch.no_grad()
    def prefill(self, prompts: list[list[int]], rows: list[int], st: KVState, left_pad: bool = True) -> Tensor:
        """Packed prefill of whole prompts into cache rows `rows` (reference: prefill_packed_host, fast_decode.py:210-269):
        the real tokens of all prompts run back to back through the trunk with causal (and, on local layers, windowed)
        attention over their own unquantized K/V; only the cache write quantises.  left_pad keeps the reference's
        positions (token j of a prompt of length n sits at T - n + j, T = longest prompt of the call) so the cache
        layout equals the reference's; left_pad=False starts every prompt at position 0.  Sets st.pos / st.starts of the
        rows and returns the final normed hidden of each prompt's last token (len(prompts), d)."""
        pk = self.pack_prompts(prompts, rows, st.max_len, left_pad)
        N, b, cfg = pk["N"], self.buf, self.cfg

        def attn(l, q):
            return self.prompt_attention(l, q, N, pk["cu"])

        h = self._trunk(pk["tok"], pk["pos"], N, attn, rows=pk["row"], last_pos=pk["last"], st=st)
        self.bind_prompts(pk, st)
        return h.index_select(0, pk["last_idx"])

    # ------------------------------------------------------------------------------------------------ generation
    @torch.no_grad()
    def generate(self, prompts: list[list[int]], max_new: int, temperature: float = 0.0, seed: int = 0,
                 max_len: int | None = None, use_graph: bool = False, return_logp: bool = False, top_k: int = 0,
                 top_p: float = 1.0, kv_dtype: str = "int8"):
        """Static-batch generation (reference: generate, model.py:1228-1263): packed prefill of all prompts, then
        lockstep decode.  temperature <= 0: greedy.  Otherwise the fused sampler with Philox uniforms keyed by
        (seed, request = prompt index, token index), truncated by top_k / top_p as sample() does (model.py:1200-1209)."""
        cfg, dev = self.cfg, self.device
        B = len(prompts)
        T = max(len(p) for p in prompts)
        st = KVState(cfg, B, max_len or (T + max_new), dev, kv_dtype=kv_dtype, dtype=self.dtype)
        req = torch.arange(B, dtype=torch.long, device=dev)
        ti = torch.zeros(B, dtype=torch.long, device=dev)

        def draw(hidden):
            xh = self.head(hidden)
            if temperature <= 0:
                return greedy_sample(xh, cfg.softcap)
            return fused_sample_seeded(xh, seed, req, ti, cfg.softcap, temperature, top_k=top_k, top_p=top_p)

        tok, lp = draw(self.prefill(prompts, list(range(B)), st))
        toks, lps = [tok.clone()], [lp.clone()]
        cur = tok.clone()
        graph = None

        def step():
            ti.add_(1)
            t, l_ = draw(self.decode_step(cur, st))
            cur.copy_(t)
            lpbuf.copy_(l_)

        lpbuf = torch.zeros(B, dtype=torch.float32, device=dev)
        for i in range(max_new - 1):
            if use_graph:
                if graph is None:
                    pos0, ti0, cur0 = st.pos.clone(), ti.clone(), cur.clone()
                    s = torch.cuda.Stream()
                    s.wait_stream(torch.cuda.current_stream())
                    with torch.cuda.stream(s):
                        step()
                    torch.cuda.current_stream().wait_stream(s)
                    st.pos.copy_(pos0); ti.copy_(ti0); cur.copy_(cur0)
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        step()
                    st.pos.copy_(pos0); ti.copy_(ti0); cur.copy_(cur0)
                graph.replay()
            else:
                step()
            toks.append(cur.clone())
            lps.append(lpbuf.clone())
        out = torch.stack(toks, 1).tolist()
        if return_logp:
            return out, torch.stack(lps, 1).cpu().numpy()
        return out
