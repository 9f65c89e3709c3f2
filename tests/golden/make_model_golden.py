"""Write tests/golden/model_golden.npz from the reference's own model code (run once, in the build container only).

Only the UV-50M forward numerics need this: nothing else pins a restatement that is consistently wrong (RoPE pairing,
rms_norm eps, XSA sign, gate slice widths, value-embedding layer set, lambda placement).  The script imports the
reference from /root/reference, builds MathLM on a reduced uv-50m-alpha shape with parameters from THIS repo's seeded
generator, runs its kernel-int8 state on the CPU (padded prefill_fast + decode_step_fast, with the GPU-only
decode_attention call replaced by the reference's own decode_attention_ref) and stores inputs and outputs as arrays.
The reference itself is never copied: the fixture holds data only.

    python tests/golden/make_model_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, "/root/reference")

from ultraviolet.kernels import fast_decode  # noqa: E402
from ultraviolet.kernels.decode_attn import decode_attention_ref  # noqa: E402
from ultraviolet.model import MathLM, make_config as ref_make_config  # noqa: E402

from ultraviolet_amd.engine.config import make_config  # noqa: E402
from ultraviolet_amd.engine.weights import random_params  # noqa: E402

SEED, PERTURB, WINDOW, MAX_LEN, STEPS = 0, 0.06, 16, 64, 24


def main():
    cfg = make_config("uv-test", window=WINDOW)
    params = random_params(cfg, SEED, perturb=PERTURB)
    rcfg = ref_make_config("uv-50m-alpha", vocab_size=cfg.vocab_size, n_layers=cfg.n_layers, d_model=cfg.d_model,
                           d_ff=cfg.d_ff, window=WINDOW)
    m = MathLM(rcfg)
    sd = m.state_dict()
    assert set(sd) == set(params), (set(sd) ^ set(params))
    m.load_state_dict({k: torch.as_tensor(np.asarray(v)).reshape(sd[k].shape) for k, v in params.items()})
    m = m.float().eval().fuse_for_inference(torch.float32)

    def attn_on_cpu(q, k_cache, v_cache, pos, starts, scale, *, window=0, ring=None, k_scale=None, v_scale=None, **_):
        return decode_attention_ref(q, k_cache, v_cache, pos, starts, scale, window=window, ring=ring, k_scale=k_scale,
                                    v_scale=v_scale)

    fast_decode.decode_attention = attn_on_cpu
    rng = np.random.default_rng(SEED)
    lens = [5, 12, 9, 20, 1, 17]
    prompts = [rng.integers(1, cfg.vocab_size, size=n).tolist() for n in lens]
    B, T = len(prompts), max(lens)
    cont = rng.integers(1, cfg.vocab_size, size=(B, STEPS))
    idx = torch.zeros(B, T, dtype=torch.long)
    starts = torch.zeros(B, dtype=torch.long)
    for b, p in enumerate(prompts):
        idx[b, T - len(p):] = torch.as_tensor(p)
        starts[b] = T - len(p)
    st = fast_decode.KernelDecodeState(rcfg, B, MAX_LEN, torch.float32, torch.device("cpu"), kv_dtype="int8")
    with torch.no_grad():
        outs = [fast_decode.prefill_fast(m, idx, starts, st)]
        for t in range(STEPS):
            outs.append(fast_decode.decode_step_fast(m, torch.as_tensor(cont[:, t]), st, MAX_LEN))
    pr = np.full((B, T), -1, np.int64)
    for b, p in enumerate(prompts):
        pr[b, :len(p)] = p
    out = dict(seed=SEED, perturb=PERTURB, window=WINDOW, max_len=MAX_LEN, prompts=pr, cont=cont,
               logits=torch.stack(outs, 1).numpy().astype(np.float32), pos=st.pos.numpy(), starts=st.starts.numpy())
    for l in range(cfg.n_layers):
        out[f"k{l}"], out[f"v{l}"] = st.k[l].numpy(), st.v[l].numpy()
        out[f"ks{l}"], out[f"vs{l}"] = st.k_scale[l].numpy(), st.v_scale[l].numpy()
    np.savez_compressed(os.path.join(HERE, "model_golden.npz"), **out)
    print("wrote model_golden.npz", {k: getattr(v, "shape", v) for k, v in out.items() if not k[0] in "kv"})


if __name__ == "__main__":
    main()
