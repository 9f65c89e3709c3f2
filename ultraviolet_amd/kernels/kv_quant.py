"""int8 KV cache: symmetric per-token-per-head quantization (absmax / 127) with fp16 scales, on the GPU.

Mirror of ultraviolet/kernels/kv_quant.py of the reference.  Cache layout: values (B, K, S, hd) int8, scales (B, K, S)
fp16; flat index of slot s of row b, kv head h is (b*K + h)*S + s for both tensors."""
from __future__ import annotations

import ctypes as C

import torch
from torch import Tensor

from .. import _lib as L


def _rows2d(x: Tensor) -> Tensor:
    """View x as (n_rows, hd) with unit inner stride and a single row stride (copy only if needed)."""
    hd = x.size(-1)
    if x.dim() == 2 and x.stride(1) == 1:
        return x
    if not x.is_contiguous():
        x = x.contiguous()
    return x.view(-1, hd)


def quantize_kv(x: Tensor) -> tuple[Tensor, Tensor]:
    """x (..., hd) float -> (int8 (..., hd), fp16 scale (...)); quantizes with the fp16-rounded scale
    (reference: kv_quant.py:12-19).  Bit-exact with the reference."""
    L.require_cuda(x)
    hd = x.size(-1)
    x2 = _rows2d(x)
    n = x2.size(0)
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(x.shape[:-1], dtype=torch.float16, device=x.device)
    if n:
        rc = L.lib().uvmi_quantize_rows(x2.data_ptr(), L.dtype_code(x2.dtype), n, hd, x2.stride(0), q.data_ptr(),
                                        s.data_ptr(), L.stream_ptr(x))
        L.check(rc, "uvmi_quantize_rows")
    return q, s


def dequantize_kv(q: Tensor, s: Tensor, dtype=torch.float16) -> Tensor:
    """reference: kv_quant.py:22-23."""
    L.require_cuda(q, s)
    q2, s2 = q.contiguous(), s.contiguous()
    out = torch.empty(q.shape, dtype=dtype, device=q.device)
    n = s2.numel()
    if n:
        rc = L.lib().uvmi_dequantize_rows(q2.data_ptr(), s2.data_ptr(), n, q.size(-1), out.data_ptr(),
                                          L.dtype_code(dtype), L.stream_ptr(q))
        L.check(rc, "uvmi_dequantize_rows")
    return out


def kv_write(cache: Tensor, scale: Tensor | None, flat_idx: Tensor, x: Tensor) -> None:
    """Decode-time write of one token per (row, kv head).  cache (B, K, S, hd) fp16/bf16 or int8; scale (B, K, S) fp16
    or None; flat_idx (B*K,) = (b*K + h)*S + slot; x (B*K, hd) or anything reshapeable to it
    (reference: kv_quant.py:26-36).  One fused quantize+scatter launch."""
    L.require_cuda(cache, flat_idx, x)
    hd = cache.size(-1)
    assert cache.is_contiguous(), "kv_write needs a contiguous cache (it is addressed through its flat view)"
    assert scale is None or scale.is_contiguous()
    x2 = _rows2d(x.reshape(-1, hd))
    n = x2.size(0)
    assert flat_idx.numel() == n and flat_idx.is_contiguous()
    rc = L.lib().uvmi_kv_write(cache.data_ptr(), L.dtype_code(cache.dtype), None if scale is None else scale.data_ptr(),
                               cache.numel() // hd, flat_idx.data_ptr(), L.dtype_code(flat_idx.dtype), x2.data_ptr(),
                               L.dtype_code(x2.dtype), n, hd, x2.stride(0), L.stream_ptr(cache))
    L.check(rc, "uvmi_kv_write")


def kv_write_rows(cache: Tensor, scale: Tensor | None, new: Tensor, slots: Tensor | slice,
                  rows: Tensor | None = None) -> None:
    """Prefill-time write.  new (n, K, T', hd) float goes to cache[rows][:, :, slots] (rows None: all rows, n == B);
    quantizes when scale is given (reference: kv_quant.py:39-54).  Implemented as one flat-index scatter instead of
    the reference's gather-modify-scatter of whole cache rows: same bytes."""
    L.require_cuda(cache, new)
    B, K, S, hd = cache.shape
    n, _, Tn, _ = new.shape
    dev = cache.device
    if isinstance(slots, slice):
        slots = torch.arange(S, device=dev)[slots]
    slots = slots.to(device=dev, dtype=torch.long)
    rws = torch.arange(B, device=dev) if rows is None else rows.to(device=dev, dtype=torch.long)
    assert rws.numel() == n and slots.numel() == Tn
    bk = rws[:, None] * K + torch.arange(K, device=dev)[None, :]           # (n, K)
    flat = (bk[:, :, None] * S + slots[None, None, :]).reshape(-1)          # (n*K*T',)
    kv_write(cache, scale, flat.contiguous(), new.reshape(-1, hd))


def kv_append(k: Tensor, v: Tensor, k_cache: Tensor, v_cache: Tensor, k_scale: Tensor, v_scale: Tensor, pos: Tensor,
              *, ring: bool, rows: Tensor | None = None) -> None:
    """Fused decode-time append of one layer's K and V (B, K, hd) at slot pos[b] (linear) or pos[b] % S (ring) of the
    int8 caches (B, K, S, hd) and fp16 scales (B, K, S): the two kv_write calls of the reference's decode step
    (fast_decode.py:291-294, 315-317) in one launch, slot arithmetic included."""
    L.require_cuda(k, v, k_cache, pos)
    B, K, S, hd = k_cache.shape
    k = k.reshape(-1, K, hd)
    v = v.reshape(-1, K, hd)
    n = k.size(0)
    assert v.shape == k.shape and k.stride() == v.stride() and k.stride(-1) == 1
    assert k_cache.stride() == v_cache.stride() and k_cache.stride(-1) == 1
    assert k_scale.stride() == v_scale.stride() and k_scale.stride(-1) == 1
    assert pos.numel() == n and pos.is_contiguous()
    if rows is not None:
        assert rows.dtype == pos.dtype and rows.numel() == n and rows.is_contiguous()
    a = L.KvAppendArgs(k.data_ptr(), v.data_ptr(), L.dtype_code(k.dtype), k.stride(0), k.stride(1),
                       k_cache.data_ptr(), v_cache.data_ptr(), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
                       k_scale.data_ptr(), v_scale.data_ptr(), k_scale.stride(0), k_scale.stride(1),
                       pos.data_ptr(), L.dtype_code(pos.dtype), None if rows is None else rows.data_ptr(),
                       n, K, S, hd, int(bool(ring)))
    L.check(L.lib().uvmi_kv_append(C.byref(a), L.stream_ptr(k)), "uvmi_kv_append")
