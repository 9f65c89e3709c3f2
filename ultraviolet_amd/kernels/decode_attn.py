"""Split-K single-query decode attention over a static, slot-indexed KV cache (MQA/GQA, ragged per-row positions,
full-context or ring-buffer sliding-window caches, fp16/bf16 or int8 with per-token-per-head fp16 scales).

Mirror of ultraviolet/kernels/decode_attn.py of the reference (`decode_attention`, `default_splits`, the
`mathk::decode_attn` custom op); the kernels are in csrc/decode_attn.hip."""
from __future__ import annotations

import ctypes as C

import torch
from torch import Tensor

from .. import _lib as L


def default_splits(n_bk: int, ctx: int, device=None, min_chunk: int = 256, waves: int = 1) -> int:
    """Splits per (row, kv head) (reference: decode_attn.py:121-129, re-derived for MI355X).  Each (row, kv head,
    split) is one workgroup whose 4 waves stream interleaved key tiles, so a row is only cut when there are fewer rows
    than `waves` workgroups per compute unit, and never into chunks shorter than min_chunk keys."""
    if device is not None:
        with torch.cuda.device(device):
            cus = L.lib().uvmi_device_cus()
    else:
        cus = L.lib().uvmi_device_cus()
    if cus <= 0:
        raise L.UvmiError(L.lib().uvmi_last_error().decode())
    want = -(-waves * cus // max(int(n_bk), 1))
    return int(max(1, min(want, max(1, int(ctx) // min_chunk), 64)))


def supported(q: Tensor, k_cache: Tensor) -> bool:
    """True when the MFMA kernel serves this geometry (reference: decode_attn_cuda.supported,
    decode_attn_cuda.py:265-270): head_dim 64, up to 8 query heads per kv head, an int8 cache or one in the q dtype.  Other
    geometries run the generic kernel."""
    H, hd = q.shape[-2], q.shape[-1]
    G = H // k_cache.shape[1]
    return bool(q.is_cuda and hd == 64 and 1 <= G <= 8 and k_cache.dtype in (torch.int8, q.dtype)
                and q.dtype in (torch.float16, torch.bfloat16))


def build_attn_args(q, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, num_splits, out, chunk_keys=0,
                    rows=None, post=None, fuse=None):
    """Fill a uvmi_attn_args struct for these tensors.  Returns (args, keepalive): the struct holds raw pointers, so the
    caller keeps `keepalive` (and the tensors) alive until the launch has been enqueued."""
    B, H, hd = q.shape
    KH, S = k_cache.shape[1], k_cache.shape[2]
    int8 = k_cache.dtype == torch.int8
    assert q.stride(-1) == 1 and k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1 and out.stride(-1) == 1
    if int8:
        assert k_scale is not None and v_scale is not None and k_scale.stride(-1) == 1 and v_scale.stride(-1) == 1
    assert pos.dtype == starts.dtype and pos.is_contiguous() and starts.is_contiguous()
    ws, ws_bytes = None, 0
    if num_splits > 1:
        ws_bytes = L.lib().uvmi_decode_attn_workspace_bytes(B, H, KH, hd, num_splits)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    a = L.AttnArgs()
    a.q, a.q_dtype, a.sqb, a.sqh = q.data_ptr(), L.dtype_code(q.dtype), q.stride(0), q.stride(1)
    a.k_cache, a.v_cache, a.kv_dtype = k_cache.data_ptr(), v_cache.data_ptr(), L.dtype_code(k_cache.dtype)
    a.skb, a.skh, a.sks = k_cache.stride(0), k_cache.stride(1), k_cache.stride(2)
    a.svb, a.svh, a.svs = v_cache.stride(0), v_cache.stride(1), v_cache.stride(2)
    if int8:
        a.k_scale, a.v_scale = k_scale.data_ptr(), v_scale.data_ptr()
        a.ssb, a.ssh, a.stb, a.sth = k_scale.stride(0), k_scale.stride(1), v_scale.stride(0), v_scale.stride(1)
    a.pos, a.starts, a.idx_dtype = pos.data_ptr(), starts.data_ptr(), L.dtype_code(pos.dtype)
    if rows is not None:
        assert rows.dtype == pos.dtype and rows.is_contiguous() and rows.numel() == B
        a.rows = rows.data_ptr()
    a.out, a.out_dtype, a.sob, a.soh = out.data_ptr(), L.dtype_code(out.dtype), out.stride(0), out.stride(1)
    a.B, a.H, a.KH, a.S, a.hd = B, H, KH, S, hd
    a.scale, a.window, a.ring, a.num_splits = float(scale), int(window), int(bool(ring)), int(num_splits)
    a.chunk_keys = int(chunk_keys)
    a.workspace, a.workspace_bytes = (ws.data_ptr() if ws is not None else None), ws_bytes
    if post is not None:
        vhat, gate, xsa, round_dtype = post
        assert vhat.dtype == torch.float32 and vhat.is_contiguous()
        a.post_vhat, a.post_round_dtype = vhat.data_ptr(), L.dtype_code(round_dtype)
        if gate is not None:
            assert gate.dtype == torch.float32 and gate.is_contiguous()
            a.post_gate = gate.data_ptr()
        if xsa is not None:
            assert xsa.dtype == torch.float32 and xsa.is_contiguous()
            a.post_xsa = xsa.data_ptr()
    f = None
    if fuse is not None:
        # fuse: dict(qkv (B, row) projection output, ext_col, has_gate, tok, ve_table, vocab, rope_table, n_pairs, rope, eps, xsa_eps)
        qkv = fuse["qkv"]
        assert qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.dtype == q.dtype
        f = L.AttnQkvFuse()
        f.qkv, f.row_stride, f.ext_col, f.has_gate = qkv.data_ptr(), qkv.stride(0), int(fuse["ext_col"]), int(bool(fuse["has_gate"]))
        ve, tok = fuse.get("ve_table"), fuse.get("tok")
        if ve is not None:
            assert tok is not None and tok.dtype == pos.dtype and tok.is_contiguous() and ve.is_contiguous() and ve.dtype == q.dtype
            f.tok, f.ve_table, f.vocab, f.has_ve = tok.data_ptr(), ve.data_ptr(), int(fuse["vocab"]), 1
        f.n_pairs, f.rope = int(fuse["n_pairs"]), int(bool(fuse["rope"]))
        if f.rope:  # (positions, 2 * n_pairs) fp32 from rope_table(): every pos must lie inside it
            tab = fuse["rope_table"]
            assert tab.dtype == torch.float32 and tab.is_contiguous() and tab.dim() == 2 and tab.size(1) == 2 * f.n_pairs
            f.rope_table, f.rope_positions = tab.data_ptr(), tab.size(0)
        f.eps, f.xsa_eps = float(fuse["eps"]), float(fuse["xsa_eps"])
        a.fuse = C.addressof(f)
    return a, (ws, rows, f)


def _launch(q, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, num_splits, out, chunk_keys=0, rows=None,
            post=None, fuse=None):
    a, keep = build_attn_args(q, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, num_splits, out, chunk_keys,
                              rows, post, fuse)
    L.check(L.lib().uvmi_decode_attn(C.byref(a), L.stream_ptr(q)), "uvmi_decode_attn")
    del keep
    return out


@torch.library.custom_op("uvmi::decode_attn", mutates_args=())
def _decode_attn_op(q: Tensor, k_cache: Tensor, v_cache: Tensor, pos: Tensor, starts: Tensor, scale: float,
                    window: int, ring: bool, k_scale: Tensor | None, v_scale: Tensor | None, num_splits: int,
                    out_fp32: bool, chunk_keys: int, rows: Tensor | None) -> Tensor:
    out = torch.empty(q.shape, device=q.device, dtype=torch.float32 if out_fp32 else q.dtype)
    return _launch(q, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, num_splits, out, chunk_keys, rows)


@_decode_attn_op.register_fake
def _(q, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, num_splits, out_fp32, chunk_keys, rows):
    return torch.empty(q.shape, device=q.device, dtype=torch.float32 if out_fp32 else q.dtype)


def _register_reference_op():
    """The reference registers its op as mathk::decode_attn (ultraviolet/kernels/decode_attn.py:174-190); code that calls
    torch.ops.mathk.decode_attn directly finds the HIP path under the same name and signature (block_n, num_warps and
    backend are accepted and ignored).  Skipped when the name is already taken (the reference imported in the same process)."""
    try:
        @torch.library.custom_op("mathk::decode_attn", mutates_args=())
        def op(q: Tensor, k_cache: Tensor, v_cache: Tensor, pos: Tensor, starts: Tensor, scale: float, window: int, ring: bool,
               k_scale: Tensor | None, v_scale: Tensor | None, num_splits: int, block_n: int, num_warps: int, backend: str) -> Tensor:
            out = torch.empty(q.shape, device=q.device, dtype=q.dtype)
            return _launch(q, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, num_splits, out)

        @op.register_fake
        def _(q, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, num_splits, block_n, num_warps, backend):
            return torch.empty_like(q)
        return op
    except RuntimeError:
        return None


_reference_op = _register_reference_op()


def decode_attention(q: Tensor, k_cache: Tensor, v_cache: Tensor, pos: Tensor, starts: Tensor, scale: float, *,
                     window: int = 0, ring: bool | None = None, k_scale: Tensor | None = None,
                     v_scale: Tensor | None = None, ctx_hint: int | None = None, num_splits: int | None = None,
                     block_n: int | None = None, num_warps: int = 1, backend: str = "auto",
                     out_fp32: bool = False, chunk_keys: int = 0, rows: Tensor | None = None) -> Tensor:
    """Single-query attention for every row of a static KV cache (reference: decode_attn.py:193-230).

    q        (B, H, hd) fp16 or bf16 (any (B, 1, H, hd) view is accepted); H = K * G, query head h*G+g uses kv head h.
    k_cache, v_cache  (B, K, S, hd) fp16/bf16, or int8 with k_scale / v_scale (B, K, S) fp16.
    pos      (B,) int: position of the current (last) key, already written to the cache.  Keys attended:
             positions max(starts[b], pos[b] - window + 1, 0) .. pos[b] (window 0 = unlimited).
    starts   (B,) int: first valid (non-pad) position of each row.
    ring     slot of position t is t % S (default: window > 0); else slot t (needs pos < S).
    ctx_hint static upper bound on keys per row (e.g. g_len, or the window) for choosing num_splits.
    block_n, num_warps, backend  accepted for signature compatibility; the HIP kernels choose their own tiling
             ("hip" / "auto" / "cuda" / "triton" all run the HIP path).
    out_fp32 return the fp32 result before rounding to q.dtype (for parity checks).
    rows     optional (B,) cache row of each query row (a compacted batch of active slots over a larger cache; a negative
             entry marks a padding row, which gets zeros).
    chunk_keys  0: every row is cut into num_splits equal chunks (the reference's rule); > 0: chunks of at least this
             many keys and at most num_splits of them per row, so short rows take fewer work items.
    Returns (B, H, hd) in q.dtype.  Graph-capturable; registered as a torch custom op (opaque to torch.compile)."""
    if q.dim() == 4:
        q = q.reshape(q.size(0), q.size(-2), q.size(-1))
    L.require_cuda(q, k_cache, v_cache, pos, starts)
    B, H, hd = q.shape
    KH, S = k_cache.shape[1], k_cache.shape[2]
    if ring is None:
        ring = window > 0
    if rows is not None:
        rows = rows.to(pos.dtype).contiguous()
    if num_splits is None:
        ctx = ctx_hint or S
        if window > 0:
            ctx = min(ctx, window)
        num_splits = default_splits(B * KH, ctx, q.device)
    q = q.contiguous() if q.stride(-1) != 1 else q
    if pos.dtype != starts.dtype:
        starts = starts.to(pos.dtype)
    return _decode_attn_op(q, k_cache, v_cache, pos.contiguous(), starts.contiguous(), float(scale), int(window),
                           bool(ring), k_scale, v_scale, int(num_splits), bool(out_fp32), int(chunk_keys), rows)


def decode_attention_post(q: Tensor, k_cache: Tensor, v_cache: Tensor, pos: Tensor, starts: Tensor, scale: float, *,
                          window: int, ring: bool, k_scale: Tensor, v_scale: Tensor, vhat: Tensor, gate: Tensor | None,
                          xsa: Tensor | None, out: Tensor, rows: Tensor | None = None) -> Tensor:
    """decode_attention followed by the reference's Attention.post up to the output projection (XSA with the
    unquantized current v, per-head sigmoid gate; ultraviolet/model.py:321-333) in the same kernel.  vhat (B, K, hd) fp32
    is v / max(|v|, eps) and gate (B, H) fp32 the gate values, both produced by the qkv_post kernel; out (B, H, hd) in
    the activation dtype is written in place.  int8 cache or a cache in the q dtype, head_dim 64, one chunk per row."""
    L.require_cuda(q, k_cache, pos)
    if rows is not None:
        rows = rows.to(pos.dtype).contiguous()
    return _launch(q, k_cache, v_cache, pos.contiguous(), starts.contiguous(), float(scale), int(window), bool(ring), k_scale,
                   v_scale, 1, out, 0, rows, (vhat, gate, xsa, out.dtype))


def rope_table(inv_freq: Tensor, n_positions: int, round_dtype: torch.dtype) -> Tensor:
    """(n_positions, 2 * n_pairs) fp32: cos(p * inv_freq) then sin(p * inv_freq), each rounded to round_dtype - the
    rotation table the fused decode path reads (the reference's Rotary buffers, ultraviolet/model.py:198-226)."""
    assert inv_freq.dtype == torch.float32 and inv_freq.is_contiguous() and inv_freq.is_cuda
    out = torch.empty(n_positions, 2 * inv_freq.numel(), dtype=torch.float32, device=inv_freq.device)
    rc = L.lib().uvmi_rope_table(inv_freq.data_ptr(), inv_freq.numel(), n_positions, L.dtype_code(round_dtype), out.data_ptr(),
                                 L.stream_ptr(inv_freq))
    L.check(rc, "uvmi_rope_table")
    return out


def decode_attention_fused(qkv: Tensor, H: int, k_cache: Tensor, v_cache: Tensor, pos: Tensor, starts: Tensor, scale: float, *,
                           window: int, ring: bool, k_scale: Tensor, v_scale: Tensor, xsa: Tensor | None, out: Tensor,
                           fuse: dict, rows: Tensor | None = None) -> Tensor:
    """A decode step's attention straight from the projection output: the kernel normalises and rotates q and k of each
    row's token, adds the value embedding to v, appends k and v to the cache at pos (int8 codes and scales, or the values
    themselves on a cache of the activation type), attends lo..pos and applies
    the XSA / gate epilogue (ultraviolet/model.py:302-333, kernels/fast_decode.py:291-325 of the reference in one launch).
    qkv (B, row) holds H*64 q, K*64 k, K*64 v and, from column fuse["ext_col"], the H gate logits and K value-embedding
    gate logits; see uvmi_attn_qkv_fuse in include/uvmi.h for the other entries of `fuse`.  The caches are written."""
    a, keep = build_fused_args(qkv, H, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, xsa, out, fuse, rows)
    L.check(L.lib().uvmi_decode_attn(C.byref(a), L.stream_ptr(qkv)), "uvmi_decode_attn")
    del keep
    return out


def build_fused_args(qkv, H, k_cache, v_cache, pos, starts, scale, window, ring, k_scale, v_scale, xsa, out, fuse, rows=None):
    """The uvmi_attn_args struct (and what must stay alive with it) of decode_attention_fused."""
    L.require_cuda(qkv, k_cache, pos)
    B = qkv.size(0)
    q = qkv.as_strided((B, H, 64), (qkv.stride(0), 64, 1))   # the q columns, for the shape / alignment checks
    if rows is not None:
        rows = rows.to(pos.dtype).contiguous()
    a, keep = build_attn_args(q, k_cache, v_cache, pos.contiguous(), starts.contiguous(), float(scale), int(window), bool(ring), k_scale,
                              v_scale, 1, out, 0, rows, None, dict(fuse, qkv=qkv))
    a.post_round_dtype = L.dtype_code(out.dtype)
    if xsa is not None:
        assert xsa.dtype == torch.float32 and xsa.is_contiguous()
        a.post_xsa = xsa.data_ptr()
    return a, (keep, q, xsa)
