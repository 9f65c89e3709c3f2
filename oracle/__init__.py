"""CPU oracle for the UV-50M decode path: a restatement of the reference algorithms, used only as a checker.

TEST INFRASTRUCTURE ONLY. Nothing under ``ultraviolet_amd/`` imports this package; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and there only to check or to time
the CPU path next to the GPU one. The product path fails loudly when the HIP library is missing; it never falls
back to this code.

Every function cites the reference file:line it follows (paths relative to the reference checkout).

Modules
  kv_quant      int8 per-row quantizer and cache writes          (ultraviolet/kernels/kv_quant.py)
  decode_attn   ragged single-query attention over a KV cache    (ultraviolet/kernels/decode_attn.py:233-263)
  fused_sample  softcap + inverse-CDF draw + log-prob            (ultraviolet/kernels/fused_sample.py:79-91)
  varlen_attn   packed causal/windowed attention                 (ultraviolet/kernels/varlen_attn.py:94-115)
  philox        Philox4x32-10 and the engine's (seed, request, token) -> uniform mapping (Random123 KATs)
  sched         continuous-batching slot bookkeeping simulator   (scripts/rl_stream.py:66-146, model.py:1293-1350)
  model         UV-50M forward / prefill / decode step in torch on the CPU (ultraviolet/model.py, fast_decode.py)
  uv_oracle.c   plain-C twin of kv_quant / decode_attn / fused_sample / philox (built by oracle/build.py)

Pinning status (what fixes each function besides its own formula) is listed at the top of each module.
"""
