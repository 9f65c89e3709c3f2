"""Helpers shared by the parity tests: seeded inputs and torch <-> numpy conversion for the oracle."""
import numpy as np
import torch


def to_np(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        return t.float().numpy()
    return t.numpy()


def attn_case(B, KH, G, hd, S, int8, seed=0, dtype=torch.float16, scale_mul=1.0):
    """Same construction as the reference's _case (tests/test_math_kernels.py:18-28): random q, K, V; int8 caches are
    the oracle quantizer's output.  Returns CPU tensors (q, k, v, ks, vs)."""
    from oracle import kv_quant
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, KH * G, hd, generator=g).to(dtype)
    k = (torch.randn(B, KH, S, hd, generator=g) * scale_mul).to(dtype)
    v = (torch.randn(B, KH, S, hd, generator=g) * scale_mul).to(dtype)
    if not int8:
        return q, k, v, None, None
    kq, ks = kv_quant.quantize_kv(to_np(k))
    vq, vs = kv_quant.quantize_kv(to_np(v))
    return q, torch.from_numpy(kq), torch.from_numpy(vq), torch.from_numpy(ks), torch.from_numpy(vs)


def rel_err(out: np.ndarray, ref: np.ndarray) -> float:
    """max |out - ref| / max(|ref|, floor): the 2e-3 bar is relative with an absolute floor for near-zero entries."""
    return float(np.max(np.abs(out - ref) / np.maximum(np.abs(ref), 1.0)))
