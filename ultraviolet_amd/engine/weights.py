"""Weights of the engine: seeded synthetic parameters under the reference's parameter names, and the fused inference
layout (the reference's fuse_for_inference, ultraviolet/model.py:289-300, 384-386, 661-667)."""
from __future__ import annotations

import math

import numpy as np
import torch

from .config import UVConfig, as_uvconfig


def random_params(cfg: UVConfig, seed: int = 0, perturb: float = 0.02, lively: bool = True) -> dict[str, np.ndarray]:
    """fp32 parameters keyed like the reference's state_dict.  Same init families as MathLM.reset_parameters
    (uniform +-sqrt(3)/2/sqrt(d) projections, zero output projections, N(0, 0.02) embeddings: model.py:282-287,
    377-382, 635-641), then every 2-D parameter += perturb * N(0, 1) (convention of the reference's
    tests/test_perf_fz.py:40-47, because the stock zero wo / w_down make attention dead code).  lively also draws the
    1-D parameters that stock init leaves neutral (XSA alphas, residual lambdas, qkv / o scales)."""
    g = np.random.default_rng(seed)
    d, hd, H, K, f = cfg.d_model, cfg.head_dim, cfg.n_heads, cfg.n_kv_heads, cfg.d_ff
    p: dict[str, np.ndarray] = {}

    def uni(shape, fan_in):
        b = math.sqrt(3) * 0.5 / math.sqrt(fan_in)
        return g.uniform(-b, b, size=shape).astype(np.float32)

    p["embed.weight"] = (g.standard_normal((cfg.vocab_size, d)) * cfg.init_std_embed).astype(np.float32)
    if cfg.use_ve:
        p["value_embed.weight"] = (g.standard_normal((cfg.vocab_size, K * hd)) * cfg.init_std_ve).astype(np.float32)
    for l in range(cfg.n_layers):
        a = f"blocks.{l}.attn."
        p[a + "wq"], p[a + "wk"], p[a + "wv"] = uni((H * hd, d), d), uni((K * hd, d), d), uni((K * hd, d), d)
        p[a + "wo"] = np.zeros((d, H * hd), np.float32)
        p[a + "qkv_scale"] = np.float32(1.0)
        p[a + "o_scale"] = np.float32(1.0)
        if cfg.has_ve(l):
            p[a + "ve_gate"] = np.zeros((K, cfg.ve_gate_channels), np.float32)
        if cfg.gate_ch:
            p[a + "attn_gate"] = np.zeros((H, cfg.gate_ch), np.float32)
        if cfg.xsa:
            p[a + "xsa_alpha"] = np.zeros((H,), np.float32)
        m = f"blocks.{l}.mlp."
        p[m + "w_gate"], p[m + "w_up"] = uni((f, d), d), uni((f, d), d)
        p[m + "w_down"] = np.zeros((d, f), np.float32)
        for s in ("resid_attn", "post_attn", "resid_mlp", "post_mlp"):
            p[f"blocks.{l}.{s}"] = np.float32(1.0)
    for k in sorted(p):
        if p[k].ndim == 2:
            p[k] = (p[k] + perturb * g.standard_normal(p[k].shape)).astype(np.float32)
    if lively:
        for l in range(cfg.n_layers):
            a = f"blocks.{l}.attn."
            if cfg.xsa:
                p[a + "xsa_alpha"] = (0.3 * g.standard_normal(H)).astype(np.float32)
            p[a + "qkv_scale"] = np.float32(1.0 + 0.05 * g.standard_normal())
            p[a + "o_scale"] = np.float32(1.0 + 0.05 * g.standard_normal())
            for s in ("resid_attn", "post_attn", "resid_mlp", "post_mlp"):
                p[f"blocks.{l}.{s}"] = np.float32(1.0 + 0.05 * g.standard_normal())
    return p


class UVWeights:
    """Fused device tensors.  Matrices are stored in the activation dtype; the small gate / XSA vectors stay fp32."""

    def __init__(self, cfg: UVConfig, params: dict, dtype=torch.bfloat16, device="cuda"):
        self.cfg, self.dtype, self.device = cfg, dtype, torch.device(device)
        self.embed, self.value_embed, self.layers = self._fuse(params)
        n_pairs = cfg.n_pairs
        # Rotary.inv_freq (model.py:203-205), same torch expression so the buffer is bit-identical
        self.inv_freq = ((1.0 / cfg.rope_base) ** torch.linspace(0, 1, n_pairs, dtype=torch.float32)).to(self.device) \
            if n_pairs else torch.zeros(1, device=self.device)

    @staticmethod
    def qkv_ext_rows(cfg: UVConfig) -> int:
        """Rows of the extended projection weight: q, k, v columns, then n_heads + n_kv_heads gate logits, padded to 16."""
        n = (cfg.n_heads + 2 * cfg.n_kv_heads) * cfg.head_dim + cfg.n_heads + cfg.n_kv_heads
        return (n + 15) // 16 * 16

    def _fuse(self, params: dict):
        """The reference's fuse_for_inference (model.py:289-300, 384-386) on a name -> array mapping."""
        cfg, dtype, dev = self.cfg, self.dtype, self.device

        def t(a):
            if isinstance(a, torch.Tensor):
                return a.detach().to("cpu", torch.float32)
            return torch.as_tensor(np.asarray(a), dtype=torch.float32)

        embed = t(params["embed.weight"]).to(dtype).to(dev).contiguous()
        value_embed = t(params["value_embed.weight"]).to(dtype).to(dev).contiguous() if cfg.use_ve else None
        layers = []
        for l in range(cfg.n_layers):
            a, m = f"blocks.{l}.attn.", f"blocks.{l}.mlp."
            # fuse(): cat(wq, wk, wv) * qkv_scale and wo * o_scale are formed in fp32, then cast (model.py:292-293)
            wqkv = torch.cat([t(params[a + "wq"]), t(params[a + "wk"]), t(params[a + "wv"])]) * float(params[a + "qkv_scale"])
            wo = t(params[a + "wo"]) * float(params[a + "o_scale"])
            gu = torch.cat([t(params[m + "w_gate"]), t(params[m + "w_up"])])
            L = {
                "wqkv": wqkv.to(dtype).to(dev).contiguous(),
                "wo": wo.to(dtype).to(dev).contiguous(),
                "gu": gu.to(dtype).to(dev).contiguous(),
                "down": t(params[m + "w_down"]).to(dtype).to(dev).contiguous(),
                # gates are cast to the activation dtype by fuse(); keep that rounding, store as fp32 for the kernels
                "ve_gate": t(params[a + "ve_gate"]).to(dtype).float().to(dev).contiguous() if cfg.has_ve(l) else None,
                "attn_gate": t(params[a + "attn_gate"]).to(dtype).float().to(dev).contiguous() if cfg.gate_ch else None,
                "xsa": torch.tanh(t(params[a + "xsa_alpha"])).to(dev).contiguous() if cfg.xsa else None,
            }
            if dtype in (torch.bfloat16, torch.float16):
                # Projection with the gate rows appended (decode steps): columns [q | k | v | H attention-gate logits |
                # K value-embedding gate logits | zero padding to a multiple of 16].  The gates are linear in the same
                # normed input (F.linear(x[..., :C], w), model.py:312, 330), so the GEMM forms their logits for free.
                d, C_g, C_v = cfg.d_model, cfg.gate_ch, cfg.ve_gate_channels
                ext = torch.zeros(self.qkv_ext_rows(cfg) - wqkv.size(0), d)
                if cfg.gate_ch:
                    ext[:cfg.n_heads, :C_g] = t(params[a + "attn_gate"]).to(dtype).float()
                if cfg.has_ve(l):
                    ext[cfg.n_heads:cfg.n_heads + cfg.n_kv_heads, :C_v] = t(params[a + "ve_gate"]).to(dtype).float()
                L["wqkv_ext"] = torch.cat([wqkv.to(dtype), ext.to(dtype)]).to(dev).contiguous()
                # gate and up rows interleaved in slabs of 16 for the GEMM whose epilogue is the SwiGLU (small decode steps)
                f = cfg.d_ff
                if f % 16 == 0:
                    g16 = gu.to(dtype)
                    L["gu_il"] = torch.stack([g16[:f].view(f // 16, 16, d), g16[f:].view(f // 16, 16, d)], 1).reshape(2 * f, d) \
                        .to(dev).contiguous()
            # the four residual scalars are cast to the activation dtype before use (model.py:568-571)
            for s in ("resid_attn", "post_attn", "resid_mlp", "post_mlp"):
                L[s] = float(torch.tensor(float(params[f"blocks.{l}.{s}"])).to(dtype).float())
            layers.append(L)
        return embed, value_embed, layers

    @torch.no_grad()
    def load_(self, params: dict) -> bool:
        """Refresh every fused tensor in place from new parameters (same names and shapes), keeping device addresses, as
        the reference's sync_weights_inplace does for its fused weights (scripts/rl_stream.py:22-36).  Returns True when
        one of the residual scalars changed: those are launch arguments, so graphs captured earlier must be recaptured."""
        embed, value_embed, layers = self._fuse(params)
        self.embed.copy_(embed)
        if self.value_embed is not None:
            self.value_embed.copy_(value_embed)
        scalars_changed = False
        self.epoch = getattr(self, "epoch", 0) + 1
        for old, new in zip(self.layers, layers):
            for k, v in new.items():
                if isinstance(v, torch.Tensor):
                    old[k].copy_(v)
                elif v is not None and old[k] != v:
                    old[k] = v
                    scalars_changed = True
        if scalars_changed:
            self.scalar_epoch = getattr(self, "scalar_epoch", 0) + 1
        return scalars_changed

    @classmethod
    def random(cls, cfg: UVConfig, seed: int = 0, dtype=torch.bfloat16, device="cuda", **kw) -> "UVWeights":
        return cls(cfg, random_params(cfg, seed, **kw), dtype, device)

    @classmethod
    def from_checkpoint(cls, ckpt: dict, dtype=torch.bfloat16, device="cuda") -> "UVWeights":
        """ckpt = {"model": state_dict, "cfg": dict} as the reference saves it (README.md:26-28).  Raises ValueError for a
        configuration with layers this engine does not implement (as_uvconfig)."""
        return cls(as_uvconfig(ckpt["cfg"]), ckpt["model"], dtype, device)

    def nbytes(self) -> int:
        n = self.embed.numel() * self.embed.element_size()
        if self.value_embed is not None:
            n += self.value_embed.numel() * self.value_embed.element_size()
        for L in self.layers:
            n += sum(v.numel() * v.element_size() for v in L.values() if isinstance(v, torch.Tensor))
        return n
