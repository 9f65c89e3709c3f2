"""End-to-end accuracy gate of the int8 KV cache: the reference's int8_check (scripts/eval_math.py:326-350) on this
engine - teacher-forced decoding of the same token rows with the unquantized cache and with the int8 cache, compared by
next-token NLL, top-1 agreement and KL divergence (published bar for the trained UV-50M: +0.002 % NLL, 99.7 % top-1)."""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor

from .model import KVState, UVEngine


@torch.no_grad()
def teacher_forced_logits(eng: UVEngine, x: Tensor, kv_dtype: str) -> Tensor:
    """Logits (B, L - 1, V) fp32 that predict x[:, 1:L], from a prefill of the first token and L - 2 decode steps fed with
    x[:, t] (eval_math.py:338-343), on a cache of the given layout ("int8", or "fp16" = unquantized in the activation type)."""
    B, L = x.shape
    st = KVState(eng.cfg, B, L + 1, eng.device, kv_dtype=kv_dtype, dtype=eng.dtype)
    out = [eng.logits(eng.prefill([[int(t)] for t in x[:, 0].tolist()], list(range(B)), st))]
    for t in range(1, L - 1):
        out.append(eng.logits(eng.decode_step(x[:, t].contiguous(), st)).clone())
    return torch.stack(out, 1).float()


@torch.no_grad()
def int8_check(eng: UVEngine, x: Tensor) -> dict:
    """x (B, L) int64 token rows on the engine's device.  Returns the reference's record: NLL per token under both caches,
    the relative change, top-1 agreement, mean KL(unquantized || int8) and the token count."""
    assert x.dim() == 2 and x.size(1) >= 3 and x.dtype == torch.int64
    lg = {kv: teacher_forced_logits(eng, x, kv) for kv in ("fp16", "int8")}
    y = x[:, 1:]
    nll = {kv: F.cross_entropy(v.transpose(1, 2), y).item() for kv, v in lg.items()}
    agree = (lg["fp16"].argmax(-1) == lg["int8"].argmax(-1)).float().mean().item()
    kl = F.kl_div(lg["int8"].log_softmax(-1), lg["fp16"].log_softmax(-1), log_target=True, reduction="none").sum(-1).mean().item()
    return {"nll_unquantized": round(nll["fp16"], 5), "nll_kernel_int8": round(nll["int8"], 5),
            "rel_change": round(nll["int8"] / nll["fp16"] - 1, 6), "top1_agree": round(agree, 5), "kl": kl,
            "tokens": int(y.numel())}
