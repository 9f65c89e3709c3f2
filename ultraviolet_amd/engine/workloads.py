"""Builders of the synthetic workloads the benchmark times and the full-size tests check: the request set of the GRPO-shaped
rollout (256 prompts x 8, geometric stop lengths), caches with materialised contexts, and the continuous-batching rollout
with per-step retirement and 64-token admissions.  Shared by bench.py and tests/test_gpu_workloads.py."""
from __future__ import annotations

import numpy as np
import torch


def c5_requests(cfg, n_prompts=256, group=8, seed=0):
    rng = np.random.default_rng(seed)
    prompts, limits = [], []
    for _ in range(n_prompts):
        n = int(rng.integers(64, 257))
        p = rng.integers(1, cfg.vocab_size, size=n).tolist()
        for _ in range(group):
            prompts.append(p)
            limits.append(int(min(rng.geometric(1.0 / 600.0), 2048)))
    return prompts, limits


def fill_cache(st, rows, ctx, gen):
    """Materialise contexts without running a prefill: random int8 K/V and fp16 scales in every cache row, pos = ctx."""
    for l in range(len(st.k)):
        for c, sc in ((st.k[l], st.k_scale[l]), (st.v[l], st.v_scale[l])):
            c.copy_(torch.randint(-127, 128, c.shape, device=c.device, dtype=torch.int8, generator=gen))
            sc.copy_((torch.rand(sc.shape, device=c.device, generator=gen) * 0.02 + 0.005).half())
    st.pos[rows] = ctx
    st.starts[rows] = 0


def c3_rollout(eng, cfg, B, n_steps, use_graph=True, seed=0, device_admit=False, check_every=4, admit_cap=24):
    """The C3 workload as a Rollout ready to step: B running slots whose contexts U{128..2048} are materialised in the cache
    (request ids 0..B-1, one token generated so far), Bernoulli(0.01) retirement per slot and step on the device, and a
    queue of 64-token prompts (ids B, B + 1, ..) long enough for n_steps steps, admitted inside decode passes."""
    from .rollout import Rollout
    dev = eng.device
    rng = np.random.default_rng(seed)
    gen = torch.Generator(device=dev).manual_seed(seed)
    g = Rollout(eng, slots=B, max_prompt=64, max_new=2048 + n_steps + 64, temperature=1.0, seed=seed, eos_id=None, check_every=check_every, bucket=128,
                retire_p=0.01, mixed=True, admit_cap=admit_cap, overlap_harvest=True, use_graph=use_graph, device_admit=device_admit)
    rows = torch.arange(B, device=dev)
    fill_cache(g.st, rows, torch.from_numpy(rng.integers(128, 2049, size=B)).to(dev), gen)
    g.slot_req.copy_(rows)
    g.slot_cnt.fill_(1)
    g.slot_limit.fill_(g.max_new)
    g.slot_tok.copy_(torch.from_numpy(rng.integers(1, cfg.vocab_size, size=B)).to(dev))
    g.free, g.next_req, g.n_active_host = [], B, B
    if device_admit:
        g.n_free_dev = 0
    for r in range(B):
        g.meta[r] = (r, 0)
    for i in range(int(n_steps * B * 0.01 * 2) + 64):
        g.add(rng.integers(1, cfg.vocab_size, size=64).tolist(), B + i)
    return g
