"""UV-50M inference path restated with torch on the CPU (checker only; see oracle/__init__.py).

What is restated, and where it comes from in the reference:
  layer math      Attention.qkv / post (ultraviolet/model.py:302-335), MLP (:388-391), Block.finish (:567-571),
                  Rotary / apply_rope (:198-226), rms_norm (:190-191), MathLM.logits (:824-827), fuse (:289-300, 384-386)
  padded prefill  MathLM.trunk with key_valid masks (:742-822) + prefill_fast cache writes (fast_decode.py:70-115)
  decode step     decode_step_fast (fast_decode.py:272-334) with decode_attention replaced by the numpy oracle
                  decode_attention_ref (there is no CPU int8 entry point in the reference: its kernel is GPU-only)
  greedy loop     generate (model.py:1228-1263) without graphs

torch is used on purpose for the float math: the reference's arithmetic for this path lives in torch library routines
(F.linear, F.rms_norm, sigmoid, softmax), and calling the same routines on the CPU restates it more faithfully than a
numpy re-derivation would.  The int8 cache, the index arithmetic and the decode attention are the numpy oracle.

Pinned by: internal invariants (prefill + decode == full forward, left-pad invariance, logits in (0, a): the reference's
tests/test_math_model.py:29-30, 73-106) in tests/test_oracle_model.py, and by the golden vectors written from the
reference itself by tests/golden/make_model_golden.py (logits and int8 cache bytes on a reduced preset).
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F

from . import decode_attn, kv_quant


def _rms(x: torch.Tensor) -> torch.Tensor:
    return F.rms_norm(x, (x.size(-1),))  # eps = finfo(x.dtype).eps, weightless (model.py:190-191)


class OracleState:
    """int8 caches as numpy arrays; same shapes as KernelDecodeState (fast_decode.py:21-57)."""

    def __init__(self, cfg, B: int, max_len: int):
        self.cfg, self.B, self.max_len = cfg, B, max_len
        self.local_len = min(cfg.window, max_len)
        self.k, self.v, self.ks, self.vs = [], [], [], []
        for l in range(cfg.n_layers):
            S = max_len if cfg.is_global(l) else self.local_len
            self.k.append(np.zeros((B, cfg.n_kv_heads, S, cfg.head_dim), np.int8))
            self.v.append(np.zeros((B, cfg.n_kv_heads, S, cfg.head_dim), np.int8))
            self.ks.append(np.zeros((B, cfg.n_kv_heads, S), np.float16))
            self.vs.append(np.zeros((B, cfg.n_kv_heads, S), np.float16))
        self.pos = np.zeros(B, np.int64)
        self.starts = np.zeros(B, np.int64)


class OracleModel:
    def __init__(self, cfg, params: dict, dtype=torch.float32):
        """params: fp32 arrays under the reference's parameter names.  dtype: the activation / weight dtype the run
        emulates (float32, or bfloat16 / float16 to follow the reference's rounding points on the CPU)."""
        self.cfg, self.dtype = cfg, dtype
        t = lambda a: torch.as_tensor(np.asarray(a), dtype=torch.float32)
        self.embed = t(params["embed.weight"]).to(dtype)
        self.value_embed = t(params["value_embed.weight"]).to(dtype) if cfg.use_ve else None
        self.layers = []
        for l in range(cfg.n_layers):
            a, m = f"blocks.{l}.attn.", f"blocks.{l}.mlp."
            Lw = {
                "wqkv": (torch.cat([t(params[a + "wq"]), t(params[a + "wk"]), t(params[a + "wv"])]) * float(params[a + "qkv_scale"])).to(dtype),
                "wo": (t(params[a + "wo"]) * float(params[a + "o_scale"])).to(dtype),
                "gu": torch.cat([t(params[m + "w_gate"]), t(params[m + "w_up"])]).to(dtype),
                "down": t(params[m + "w_down"]).to(dtype),
                "ve_gate": t(params[a + "ve_gate"]).to(dtype) if cfg.has_ve(l) else None,
                "attn_gate": t(params[a + "attn_gate"]).to(dtype) if cfg.gate_ch else None,
                "xsa": torch.tanh(t(params[a + "xsa_alpha"])) if cfg.xsa else None,
            }
            for s in ("resid_attn", "post_attn", "resid_mlp", "post_mlp"):
                Lw[s] = torch.tensor(float(params[f"blocks.{l}.{s}"])).to(dtype)
            self.layers.append(Lw)
        self.inv_freq = (1.0 / cfg.rope_base) ** torch.linspace(0, 1, cfg.n_pairs, dtype=torch.float32) if cfg.n_pairs else None

    # ---- pieces -------------------------------------------------------------------------------------------
    def _cos_sin(self, pos: torch.Tensor):
        th = pos.float()[..., None] * self.inv_freq
        return th.cos(), th.sin()

    def _rope(self, x, cos, sin):
        """x (B, T, H, hd); cos / sin (B, T, n_pairs).  Half-split pairing on the first 2 * n_pairs dims."""
        n = self.cfg.n_pairs
        c, s = cos.unsqueeze(-2).to(x.dtype), sin.unsqueeze(-2).to(x.dtype)
        x1, x2, rest = x[..., :n], x[..., n:2 * n], x[..., 2 * n:]
        return torch.cat([x1 * c - x2 * s, x1 * s + x2 * c, rest], dim=-1)

    def _qkv(self, l, xn, ve, cos, sin):
        cfg, W = self.cfg, self.layers[l]
        B, T, _ = xn.shape
        H, K, hd = cfg.n_heads, cfg.n_kv_heads, cfg.head_dim
        q, k, v = F.linear(xn, W["wqkv"]).split([H * hd, K * hd, K * hd], dim=-1)
        q, k, v = q.view(B, T, H, hd), k.view(B, T, K, hd), v.view(B, T, K, hd)
        if cfg.has_ve(l):
            gw = W["ve_gate"]
            g = 2.0 * torch.sigmoid(F.linear(xn[..., :gw.size(-1)], gw))
            v = v + g.unsqueeze(-1) * ve.to(v.dtype)
        q, k = _rms(q), _rms(k)
        if (not cfg.is_global(l)) or cfg.global_rope:
            q, k = self._rope(q, cos, sin), self._rope(k, cos, sin)
        return q, k, v

    def _post(self, l, z, xn, v):
        cfg, W = self.cfg, self.layers[l]
        B, T = z.shape[:2]
        H, K, hd = cfg.n_heads, cfg.n_kv_heads, cfg.head_dim
        G = H // K
        if cfg.xsa:
            zg = z.view(B, T, K, G, hd).float()
            vd = F.normalize(v.float(), dim=-1, eps=cfg.xsa_eps).unsqueeze(3)
            proj = (zg * vd).sum(-1, keepdim=True)
            z = (zg - W["xsa"].view(1, 1, K, G, 1) * proj * vd).to(z.dtype).view(B, T, H, hd)
        if cfg.gate_ch:
            g = 2.0 * torch.sigmoid(F.linear(xn[..., :cfg.gate_ch], W["attn_gate"]))
            z = z * g.unsqueeze(-1).to(z.dtype)
        return F.linear(z.reshape(B, T, -1), W["wo"])

    def _finish(self, l, base, a):
        W = self.layers[l]
        h = W["resid_attn"] * base + W["post_attn"] * a
        n = _rms(h)
        g, u = F.linear(n, W["gu"]).chunk(2, dim=-1)
        m = F.linear(F.silu(g) * u, W["down"])
        return W["resid_mlp"] * h + W["post_mlp"] * m

    def logits(self, h):
        a, b, c = self.cfg.softcap
        return a * torch.sigmoid((F.linear(h, self.embed).float() + b) / c)

    def head_raw(self, h):
        return F.linear(h, self.embed)

    # ---- full-sequence trunk with left-pad masks (padded prefill) --------------------------------------------
    def trunk(self, idx: torch.Tensor, key_valid: torch.Tensor | None = None):
        """idx (B, T) -> final normed hidden (B, T, d), per-layer (k, v) each (B, T, K, hd)."""
        cfg = self.cfg
        B, T = idx.shape
        cos, sin = self._cos_sin(torch.arange(T))
        cos, sin = cos[None].expand(B, T, -1), sin[None].expand(B, T, -1)
        ve = self.value_embed[idx].view(B, T, cfg.n_kv_heads, cfg.head_dim) if cfg.use_ve else None
        x = _rms(self.embed[idx])
        i = torch.arange(T)
        dd = i[:, None] - i[None, :]
        causal, local = dd >= 0, (dd >= 0) & (dd < cfg.window)
        if key_valid is not None:  # pad keys masked; pad query rows see themselves so the softmax stays finite
            eye = torch.eye(T, dtype=torch.bool)
            kvm = key_valid[:, None, None, :]
            masks = {True: (causal & kvm) | eye, False: (local & kvm) | eye}
        else:
            masks = {True: causal[None, None], False: local[None, None]}
        G = cfg.n_heads // cfg.n_kv_heads
        kvs = []
        for l in range(cfg.n_layers):
            xn = _rms(x)
            q, k, v = self._qkv(l, xn, ve, cos, sin)
            qt, kt, vt = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
            if G > 1:
                kt, vt = kt.repeat_interleave(G, dim=1), vt.repeat_interleave(G, dim=1)
            s = (qt.float() @ kt.float().transpose(-1, -2)) * cfg.attn_scale
            s = s.masked_fill(~masks[cfg.is_global(l)], float("-inf"))
            z = (torch.softmax(s, -1) @ vt.float()).to(q.dtype).transpose(1, 2)
            x = self._finish(l, x, self._post(l, z, xn, v))
            kvs.append((k, v))
        return _rms(x), kvs

    # ---- prefill into an int8 state (left-padded, as the reference's default path) ----------------------------
    def prefill(self, prompts: list[list[int]], rows: list[int], st: OracleState):
        """Left-pad the prompts to the longest one, run the padded trunk, write the quantized K/V of the real tokens
        into cache rows `rows` (global: slot = position; ring: last S positions at slot = position % S), set
        pos = T, starts = T - len.  Returns the last-position hidden (n, d).  fast_decode.py:70-115, model.py:1214-1221."""
        cfg = self.cfg
        n = len(prompts)
        T = max(len(p) for p in prompts)
        idx = torch.zeros(n, T, dtype=torch.long)
        starts = np.zeros(n, np.int64)
        for b, p in enumerate(prompts):
            idx[b, T - len(p):] = torch.as_tensor(p)
            starts[b] = T - len(p)
        key_valid = torch.arange(T)[None, :] >= torch.as_tensor(starts)[:, None]
        h, kvs = self.trunk(idx, key_valid)
        rows_np = np.asarray(rows, np.int64)
        for l, (k, v) in enumerate(kvs):
            for cache, sc, new in ((st.k[l], st.ks[l], k), (st.v[l], st.vs[l], v)):
                S = cache.shape[2]
                nt = new.transpose(1, 2).float().numpy()  # (n, K, T, hd)
                if cfg.is_global(l):
                    kv_quant.kv_write_rows(cache, sc, nt, slice(0, T), rows_np)
                else:
                    lo = max(0, T - S)
                    kv_quant.kv_write_rows(cache, sc, nt[:, :, lo:], np.arange(lo, T) % S, rows_np)
        st.starts[rows_np] = starts
        st.pos[rows_np] = T
        return h[:, -1]

    # ---- one decode step over an int8 state --------------------------------------------------------------------
    def decode_step(self, tok: np.ndarray, st: OracleState):
        """fast_decode.py:272-334: write K/V at pos first, attend max(starts, pos - W + 1)..pos, pos += 1.
        Returns the final normed hidden (B, d)."""
        cfg = self.cfg
        B = len(tok)
        K, hd, H = cfg.n_kv_heads, cfg.head_dim, cfg.n_heads
        p = st.pos.copy()
        idx = torch.as_tensor(np.asarray(tok, np.int64)).view(B, 1)
        cos, sin = self._cos_sin(torch.as_tensor(p))
        cos, sin = cos[:, None, :], sin[:, None, :]
        ve = self.value_embed[idx].view(B, 1, K, hd) if cfg.use_ve else None
        x = _rms(self.embed[idx]).to(self.dtype)
        for l in range(cfg.n_layers):
            xn = _rms(x)
            q, k, v = self._qkv(l, xn, ve, cos, sin)
            glob = cfg.is_global(l)
            S = st.k[l].shape[2]
            ix = kv_quant.decode_flat_index(p, K, S, ring=not glob)
            kv_quant.kv_write(st.k[l], st.ks[l], ix, k.reshape(B * K, hd).float().numpy())
            kv_quant.kv_write(st.v[l], st.vs[l], ix, v.reshape(B * K, hd).float().numpy())
            z = decode_attn.decode_attention_ref(q.reshape(B, H, hd).float().numpy(), st.k[l], st.v[l], p, st.starts,
                                                 cfg.attn_scale, window=0 if glob else cfg.window, ring=not glob,
                                                 k_scale=st.ks[l], v_scale=st.vs[l])
            z = torch.from_numpy(z).to(q.dtype).view(B, 1, H, hd)
            x = self._finish(l, x, self._post(l, z, xn, v))
        st.pos += 1
        return _rms(x)[:, 0]

    # ---- greedy generation ----------------------------------------------------------------------------------------
    def generate_greedy(self, prompts: list[list[int]], max_new: int, max_len: int | None = None, return_logits=False):
        B = len(prompts)
        T = max(len(p) for p in prompts)
        st = OracleState(self.cfg, B, max_len or (T + max_new))
        lg = self.logits(self.prefill(prompts, list(range(B)), st))
        tok = lg.argmax(-1).numpy()
        out, lgs = [tok.copy()], [lg.numpy()]
        for _ in range(max_new - 1):
            lg = self.logits(self.decode_step(tok, st))
            tok = lg.argmax(-1).numpy()
            out.append(tok.copy())
            lgs.append(lg.numpy())
        toks = np.stack(out, 1)
        return (toks, np.stack(lgs, 1), st) if return_logits else toks
