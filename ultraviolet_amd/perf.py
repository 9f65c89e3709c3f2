"""The generation-side names of the reference's ultraviolet/perf.py (make_streamgen :543-570, install_fz :572-588) and of
scripts/rl_stream.py (StreamGen :39-64, sync_weights_inplace :22-36), so that rl_grpo.stream_loop's calls
(scripts/rl_grpo.py:1091-1105) find them here.

What the reference's perf flags switch on one by one is how the Rollout driver of this package always works: behaviour
log-probs come out of the sampler's launch ('lp'), the harvest copies only finished rows ('hv'), prefill index tables are
never built with device synchronisation ('rfh'), and a decode step is trunk -> head GEMM -> fused sampler ('fz').  So
make_streamgen has nothing to wrap and install_fz nothing to install: both answer for the caller's control flow."""
from __future__ import annotations

import torch

from . import _lib as L
from .engine.rollout import Rollout
from .kernels.fast_decode import _engine, _weights_stamp, patch_model, sync_patched_weights
from .kernels.fused_sample import fused_sample_ok

PERF_FLAGS = {"lp", "hv", "rfh", "fz", "acc16", "pack", "head16", "pf", "pfc", "pkv"}


class StreamGen(Rollout):
    """StreamGen(model, slots, max_prompt, max_new, temperature, eos_id, ...) of the reference (scripts/rl_stream.py:39-64)
    on the device-side slot table: add / chunk / n_active / n_outstanding / drop_queued and the (meta, tokens, logp,
    start_version) results are Rollout's.  `model` is a model patch_model has bound (or binds here, int8 KV);
    `bucket` is the reference's context-length bucket of its graphs and has no meaning here (one graph serves every
    context length); row_bucket is the granularity of the active-row buckets the step graphs are captured for."""

    def __init__(self, model, slots, max_prompt, max_new, temperature, eos_id, check_every=16, compile=True, use_graph=True,
                 pad_id=0, dtype=torch.bfloat16, bucket=1024, row_bucket=128, seed=0):
        assert temperature > 0
        if model.__dict__.get("_uvmi_engine") is None:
            patch_model(model, kv_dtype="int8", dtype=dtype, max_tokens=max(16384, slots))
        self.m = model
        super().__init__(_engine(model), slots, max_prompt, max_new, temperature=temperature, seed=seed, eos_id=eos_id,
                         check_every=check_every, bucket=min(row_bucket, slots), use_graph=use_graph, left_pad=True)

    def chunk(self):
        """StreamGen.chunk of the reference.  Parameters the trainer has written in place since the last chunk are brought
        into the engine first (the reference's graphs read the live fused weights); `version` is left alone - it is the
        caller's counter (scripts/rl_grpo.py:1309)."""
        if _weights_stamp(self.m) != self.m.__dict__.get("_uvmi_stamp"):
            sync_patched_weights(self.m)
            torch.cuda.synchronize(self.dev)
        self._check_weight_epoch()
        return super().chunk()


def make_streamgen(base, flags):
    """The reference returns a subclass of `base` with the flags' fast paths (perf.py:543-570); here `base` already has
    them all, so it is returned as is.  Unknown flags raise, as a typo would silently cost the reference its speed-up."""
    bad = set(flags) - PERF_FLAGS
    if bad:
        raise L.UvmiError(f"unknown perf flags {sorted(bad)}")
    if not (isinstance(base, type) and issubclass(base, Rollout)):
        raise L.UvmiError("make_streamgen expects this package's StreamGen / Rollout class")
    return base


def install_fz(runner) -> bool:
    """Whether the runner's decode step draws its tokens with the fused sampler (perf.py:572-588).  True for a Rollout /
    StreamGen with temperature > 0 whose vocabulary and softcap the sampler covers; nothing is replaced - the step is
    built that way."""
    if not isinstance(runner, Rollout) or runner.T <= 0:
        return False
    cfg = runner.cfg
    return bool(fused_sample_ok(runner.dev, cfg.vocab_size, cfg.softcap, runner.T))


@torch.no_grad()
def sync_weights_inplace(gen_m, raw) -> None:
    """sync_weights_inplace(gen_m, raw) of the reference (scripts/rl_stream.py:22-36): the policy `raw` becomes the weights
    of the generation model `gen_m` - a model patch_model has bound - in place: its parameters are overwritten, and the
    engine's fused device tensors are refreshed at their addresses, so captured step graphs keep reading the same tensors.
    A StreamGen / Rollout is accepted in place of the model (its engine's weights are refreshed from raw.state_dict()).
    As in the reference, the generator's `version` is not touched: the caller advances it (scripts/rl_grpo.py:1308-1309)."""
    if isinstance(gen_m, Rollout):
        gen_m.sync_weights_inplace(raw.state_dict())
        return
    if gen_m.__dict__.get("_uvmi_engine") is None:
        raise L.UvmiError("sync_weights_inplace: the generation model has not been patched (patch_model) and is not a StreamGen")
    if gen_m is not raw:
        if hasattr(gen_m, "parameters") and hasattr(raw, "parameters"):
            for pg, pt in zip(gen_m.parameters(), raw.parameters()):
                pg.copy_(pt)
        else:
            src = raw.state_dict()
            for k, t in gen_m.state_dict().items():
                t.copy_(src[k])
    sync_patched_weights(gen_m)
    torch.cuda.synchronize(next(iter(gen_m.__dict__["_uvmi_live"])).device)
