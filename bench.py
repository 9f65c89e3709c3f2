#!/usr/bin/env python3
"""Benchmark of the UV-50M decode hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5|c2|c3|c4|copy]

Workload c5 (default; BASELINE.json configs[4], the configuration the metric is quoted on): GRPO-shaped rollout,
256 prompts x group 8 = 2048 concurrent sequences, prompt lengths U{64..256} shared inside a group, T = 1.0 with seeded
Philox sampling, per-sequence stop length min(Geom(1/600), 2048), random-init (perturbed) UV-50M in bf16 with an int8
KV cache.  All prompts are prefilled (untimed, reported separately), W decode steps run untimed, then exactly K decode
steps of the rollout are timed; a step is 10-layer trunk over the active rows -> tied head -> fused sampler -> commit,
replayed from a captured graph (the active rows are compacted again when the bucket shrinks), with the inputs resident
in HBM.  value = tokens generated in the timed steps / seconds.  With --steps K the timed window is decode steps
W .. W + K of the rollout (right after admission: nearly all 2048 slots live, the shortest contexts); the same rollout
is then run to completion and its whole-run figures are reported beside it as "full_rollout" (with --steps 0, the default,
the timed region is the whole rollout itself).

After the timed region the same rollout is replayed eagerly and, on a subsample of steps, the step's decode-attention
launches are re-issued through the C ABI between HIP events on the launch stream to get the attention kernel's average
launch duration and algorithmic bytes (132 B per attended key + q/out + positions) for the roofline object.
The cpu_baseline object times this repo's CPU restatement of the reference path (oracle/, kind "port") on a bounded
sample of the same workload on the host cores.

Other workloads (parity-test configurations, timed for reference, not the headline):
  c2    BASELINE.json configs[1]: the single-layer ragged int8-KV attention op alone, cold caches;
  c3    configs[2]: 512 slots with contexts U{128..2048}, every step each slot retires with p = 0.01 (seeded, on the
        device) and queued 64-token prompts are admitted into freed slots inside decode passes (mixed batches);
  c4    configs[3]: one forward pass over 64 prompt chunks x 512 tokens packed with 448 decode rows, contexts U{256..2048};
  copy  a 1 GiB device copy, the calibration kernel for the HBM traffic counters.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from ultraviolet_amd.engine.workloads import c3_rollout, c5_requests as _c5_requests, fill_cache as _fill_cache  # noqa: E402

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch / algorithmic bytes per launch of the decode-attention kernel, from the FETCH_SIZE and
# WRITE_SIZE counter runs summarised in profiles/c5_attention_hbm_counters.md (FETCH_SIZE scaled x2.000 and WRITE_SIZE
# x1.000 by what they read for a 1 GiB device copy).
TRAFFIC_PER_ALGORITHMIC_BYTE = 1.10


def _attn_bytes(pos, starts, window, B, H=8, hd=64):
    lo = np.maximum(starts, 0)
    if window:
        lo = np.maximum(lo, pos - window + 1)
    n = np.maximum(pos - lo + 1, 0)
    return 132 * int(n.sum()) + 4 * B * H * hd + 16 * B


def bench_c5(args):
    from ultraviolet_amd.engine import UVEngine, UVWeights, make_config
    from ultraviolet_amd.engine.rollout import Rollout
    dev = "cuda:0"
    cfg = make_config("uv-50m-alpha")
    weights = UVWeights.random(cfg, seed=0, dtype=torch.bfloat16, device=dev, perturb=0.02)
    eng = UVEngine(weights, max_tokens=16384)
    prompts, limits = _c5_requests(cfg)
    n_seq = len(prompts)

    def make_rollout(use_graph):
        g = Rollout(eng, slots=n_seq, max_prompt=256, max_new=2048, temperature=1.0, seed=0, eos_id=None, check_every=16,
                    bucket=32, use_graph=use_graph, share_prompts=True)
        for i, (p, l) in enumerate(zip(prompts, limits)):
            g.add(p, i, limit=l)
        return g

    gw = make_rollout(False)   # warm-up of the prefill path (first use loads every kernel and the GEMM library's solutions)
    gw._admit()
    del gw
    g = make_rollout(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    g._admit()
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    prefill_tokens = sum(len(p) for p in prompts)
    prefill_unique = g.n_prefill_tokens   # a group of 8 shares its prompt: prefilled once per admission call, cache rows copied
    g.precapture()
    total_steps = max(limits) - 1
    W = min(args.warmup, total_steps - 1)
    K = min(args.steps, total_steps - W) if args.steps > 0 else total_steps - W

    def run_steps(gg, n):
        """n decode steps with a harvest every check_every steps; the host takes a harvest's results after it has enqueued
        the following step, so that its share of the work costs no idle GPU time."""
        done = 0
        while done < n:
            m = min(gg.ce, n - done)
            for i in range(m):
                gg.step()
                if i == 0 and gg.harvest_pending:
                    gg.harvest_end()
            done += m
            gg.harvest_begin()
        gg.harvest_end()

    run_steps(g, W)
    torch.cuda.synchronize()
    tok0 = int(g.slot_cnt[g.slot_req >= 0].sum()) + g.n_tokens
    active0 = g.n_active()
    t0 = time.perf_counter()
    run_steps(g, K)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    tok1 = int(g.slot_cnt[g.slot_req >= 0].sum()) + g.n_tokens
    gen = tok1 - tok0
    value = gen / dt
    active1 = g.n_active()
    # ---- the rest of the same rollout, to completion: the whole-run figure next to the timed window's
    rest = total_steps - W - K
    dt_rest = 0.0
    if rest > 0:
        t0 = time.perf_counter()
        run_steps(g, rest)
        torch.cuda.synchronize()
        dt_rest = time.perf_counter() - t0
    tok2 = int(g.slot_cnt[g.slot_req >= 0].sum()) + g.n_tokens
    steps_all, dt_all = K + rest, dt + dt_rest

    # ---- roofline of the dominant kernel: replay the same steps eagerly with events around the attention calls
    roof, roof_full = roofline_c5(make_rollout, eng, cfg, W, K, total_steps - W)
    cpu = cpu_baseline_c5(cfg, prompts, limits)
    full = {"tok_per_s": round((tok2 - tok0) / dt_all, 1), "steps": steps_all, "ms_per_step": round(dt_all * 1e3 / steps_all, 4),
            "mean_active_rows": round((tok2 - tok0) / steps_all, 1), "tokens": tok2 - tok0, "active_at_end": g.n_active(),
            "roofline_frac": roof_full["frac"], "roofline_achieved_GBs": roof_full["achieved"],
            "attention_avg_launch_us": roof_full["avg_launch_us"], "attention_bytes_per_launch": roof_full["bytes_per_launch"]}
    out = {
        "metric": "decode tok/s, UV-50M ragged batch 2048", "value": round(value, 1), "unit": "tok/s", "n_gpus": 1,
        "steps": K, "warmup": W, "ms_per_step": round(dt * 1e3 / K, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C5 GRPO rollout: 256 prompts x 8 = 2048 sequences, prompts U{64..256}, T=1.0 Philox seed 0, "
                               "stop min(Geom(1/600), 2048), UV-50M (10L d640 8x64 MQA, vocab 32768) bf16, int8 KV",
                   "timed_window": f"decode steps {W}..{W + K} of {total_steps} (whole rollout)" if rest <= 0 else
                                   f"decode steps {W}..{W + K} of {total_steps}: the steps right after admission, all slots live, shortest "
                                   f"contexts; the whole rollout is in full_rollout",
                   "slots": n_seq, "active_at_start": active0, "active_at_end": active1, "tokens_timed": gen,
                   "prefill_tokens": prefill_tokens, "prefill_tokens_computed": prefill_unique, "prefill_s": round(prefill_s, 3),
                   "prefill_tok_per_s": round(prefill_unique / prefill_s, 1), "kv_cache_GB": round(g.st.nbytes() / 1e9, 3)},
        "roofline": roof, "cpu_baseline": cpu, "full_rollout": full,
    }
    print(json.dumps(out))


def roofline_c5(make_rollout, eng, cfg, W, K, K_all, every=16, reps=3):
    """Average launch duration and algorithmic bytes of the decode-attention kernel over the timed steps, by HIP events
    on the launch stream.  The same rollout is replayed eagerly; after every `every`-th timed step the step's ten
    attention launches are re-issued through the C ABI on that step's state, `reps` times back to back, between two
    events (sequence A), and likewise the eight ring-layer launches alone (sequence B).  One step's attention working set
    (~0.5 GB) exceeds the 256 MB last-level cache, so every launch streams from HBM as in the real step; re-issuing a
    single launch in a loop would be served from that cache.  Global-layer time = (A - B) / 2 per step.  The launches go
    through ctypes directly (a few microseconds each), so the host stays ahead of the GPU, and a fill kernel ahead of the
    first event keeps the queue non-empty while the sequence is enqueued.
    Returns two roofline objects: over the samples of the timed window (steps W .. W + K) and over the samples of the
    whole rollout (steps W .. W + K_all)."""
    import ctypes as C
    from ultraviolet_amd import _lib as L
    lib = L.lib()
    g = make_rollout(False)
    g._admit()
    fused = eng.fuse_qkv
    if fused:   # keep each layer's projection of the sampled step, so that the re-issued launches are the step's own
        eng.qkvx_keep = [torch.empty_like(eng.buf["qkvx"][:g.B]) for _ in range(cfg.n_layers)]
    layers = list(range(cfg.n_layers))
    ring_layers = [l for l in layers if not cfg.is_global(l)]
    n_glob = len(layers) - len(ring_layers)
    scratch = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    samples = []   # (events A, events B, bytes global, bytes ring)
    ev_plain = []  # events of the attention-only kernel's sequence A (when the step runs the fused kernel)

    def timed_seq(args_list, probe=0):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        scratch.zero_()
        e0.record()
        for _ in range(reps):
            for a in args_list:
                rc = lib.uvmi_decode_attn_probe(C.byref(a), probe, stream) if probe else lib.uvmi_decode_attn(C.byref(a), stream)
                if rc:
                    L.check(rc, "uvmi_decode_attn")
        e1.record()
        return e0, e1

    ev_probe = {1: [], 2: []}   # the attention-only launches with half of the kernel's work taken out (uvmi_decode_attn_probe)

    in_window = []
    for s in range(W + K_all):
        sampled = s >= W and (s - W) % every == 0
        if sampled:   # the step's own rows, tokens and positions (the step leaves the next step's in their place)
            n, act, tok, pos, starts = (t if isinstance(t, int) else t.clone() for t in g.step_inputs())
        g.step()
        if sampled:
            torch.cuda.synchronize()
            if fused:
                built = {l: eng.fused_attention_args(l, eng.qkvx_keep[l], tok, g.st, pos, starts, n, rows=act) for l in layers}
            else:
                built = {l: eng.cache_attention_args(l, g.st, pos, starts, n, rows=act) for l in layers}
            evA = timed_seq([built[l][0] for l in layers])
            evB = timed_seq([built[l][0] for l in ring_layers])
            if fused:   # the attention-only kernel on the same caches and positions (q and the epilogue inputs are whatever
                        # the engine's buffers hold: only the timing is used)
                plain = {l: eng.cache_attention_args(l, g.st, pos, starts, n, rows=act) for l in layers}
                ev_plain.append(timed_seq([plain[l][0] for l in layers]))
                out_keep = eng.buf["zg"][:n].clone()     # (the probes write meaningless values to the layer output buffer)
                for mode in (1, 2):
                    ev_probe[mode].append(timed_seq([plain[l][0] for l in layers], probe=mode))
                eng.buf["zg"][:n].copy_(out_keep)
            torch.cuda.synchronize()
            live = act.cpu().numpy() >= 0
            p, st = pos.cpu().numpy()[live], starts.cpu().numpy()[live]   # what the kernels saw (padding rows: no keys)
            samples.append((evA, evB, _attn_bytes(p, st, 0, n), _attn_bytes(p, st, cfg.window, n)))
            in_window.append(s < W + K)
            del built
        if (s + 1) % g.ce == 0:
            g.poll()
    eng.qkvx_keep = None

    def aggregate(sel):
        smp = [x for x, k in zip(samples, sel) if k]
        evp = [x for x, k in zip(ev_plain, sel) if k] if ev_plain else []
        tA = sum(a.elapsed_time(b) for (a, b), _, _, _ in smp) * 1e3 / reps      # us, all layers, summed over samples
        tB = sum(a.elapsed_time(b) for _, (a, b), _, _ in smp) * 1e3 / reps      # us, ring layers only
        ns = len(smp)
        n_all = len(layers)
        glob_us = (tA - tB) / (n_glob * ns)
        ring_us = tB / (len(ring_layers) * ns)
        all_us = tA / (n_all * ns)
        glob_bytes = sum(x[2] for x in smp) / ns
        ring_bytes = sum(x[3] for x in smp) / ns
        all_bytes = (n_glob * glob_bytes + len(ring_layers) * ring_bytes) / n_all
        gb, rb, ab = glob_bytes / glob_us / 1e3, ring_bytes / ring_us / 1e3, all_bytes / all_us / 1e3
        # The headline figure covers every decode-attention launch of the step (sequence A as timed: two global-layer and
        # eight ring-layer launches of the same kernel); the split by layer kind (A - B, B) is reported beside it.
        extra = {}
        if evp:
            plain_us = sum(a.elapsed_time(b) for a, b in evp) * 1e3 / reps / (n_all * ns)
            extra["attention_only_kernel"] = {
                "kernel": "uvmi::attn_mfma_i8_hd64<1, 1, WPR, FUSE=false> (the same launches without the fused QKV post-processing, which then "
                          "costs a separate ~10 us launch per layer)",
                "achieved": round(all_bytes / plain_us / 1e3, 1), "frac": round(all_bytes / plain_us / 1e3 / HBM_PEAK_GBS, 4),
                "avg_launch_us": round(plain_us, 2), "launches_timed": n_all * ns * reps}
            pr = {m: sum(a.elapsed_time(b) for (a, b), k in zip(ev_probe[m], sel) if k) * 1e3 / reps / (n_all * ns) for m in (1, 2)}
            extra["ceiling_probes"] = {
                "what": "the attention-only launches re-issued through uvmi_decode_attn_probe: mode 1 keeps the kernel's memory stream and drops "
                        "its arithmetic, mode 2 keeps the arithmetic and reads no cache",
                "stream_only_us": round(pr[1], 2), "stream_only_frac": round(all_bytes / pr[1] / 1e3 / HBM_PEAK_GBS, 4),
                "arithmetic_only_us": round(pr[2], 2), "kernel_us": round(plain_us, 2)}
        return {"bound": "hbm", "achieved": round(ab, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ab / HBM_PEAK_GBS, 4),
                "traffic": int(all_bytes * TRAFFIC_PER_ALGORITHMIC_BYTE),
                "kernel": "uvmi::attn_mfma_i8_hd64<1, 1, WPR, FUSE=true> (bf16; all ten layers' launches of a step; the kernel also does the "
                          "row's QKV post-processing and int8 append; WPR = 2 waves per row while 4 would not fit the device in one round, else 4)",
                "avg_launch_us": round(all_us, 2), "bytes_per_launch": int(all_bytes), "steps_sampled": ns, "launches_timed": n_all * ns * reps,
                "global_layers": {"achieved": round(gb, 1), "frac": round(gb / HBM_PEAK_GBS, 4), "avg_launch_us": round(glob_us, 2),
                                  "bytes_per_launch": int(glob_bytes), "launches_timed": n_glob * ns * reps},
                "ring_layers": {"achieved": round(rb, 1), "frac": round(rb / HBM_PEAK_GBS, 4), "avg_launch_us": round(ring_us, 2),
                                "bytes_per_launch": int(ring_bytes), "launches_timed": len(ring_layers) * ns * reps}, **extra}

    return aggregate(in_window), aggregate([True] * len(samples))


def cpu_baseline_c5(cfg, prompts, limits, budget_s=15.0, rows=32):
    """The CPU restatement of the reference path (oracle.model, torch fp32 eager) on a bounded sample: the first `rows`
    sequences of the same workload, prefilled and then decoded greedily until the time budget is spent."""
    from oracle.model import OracleModel, OracleState
    from ultraviolet_amd.engine.weights import random_params
    params = random_params(cfg, 0, perturb=0.02)
    m = OracleModel(cfg, params, torch.float32)
    sub = prompts[:rows]
    st = OracleState(cfg, rows, 256 + 2048 + 1)
    t0 = time.perf_counter()
    tok = m.logits(m.prefill(sub, list(range(rows)), st)).argmax(-1).numpy()
    t_pre = time.perf_counter() - t0
    t0 = time.perf_counter()
    steps = 0
    while time.perf_counter() - t0 < budget_s:
        tok = m.logits(m.decode_step(tok, st)).argmax(-1).numpy()
        steps += 1
    dt = time.perf_counter() - t0
    return {"value": round(rows * steps / dt, 2), "unit": "tok/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{rows} of the 2048 sequences (prompts U{{64..256}}), fp32 eager torch CPU oracle of the reference path, "
                      f"{steps} greedy decode steps after a {t_pre:.1f} s prefill; host cpu_count={os.cpu_count()}, torch {torch.__version__}"}


def bench_c2(args):
    """BASELINE configs[1]: 256 sequences, 8 heads x 64, KH = 1, contexts U{64..1024}, bf16 q, int8 KV (cold: rotating sets)."""
    from ultraviolet_amd.kernels import decode_attention
    dev = "cuda:0"
    B, S = 256, 1024
    g = torch.Generator(device=dev).manual_seed(0)
    nsets = 32
    sets = []
    for _ in range(nsets):
        sets.append((torch.randint(-127, 128, (B, 1, S, 64), device=dev, dtype=torch.int8, generator=g),
                     torch.randint(-127, 128, (B, 1, S, 64), device=dev, dtype=torch.int8, generator=g),
                     (torch.rand(B, 1, S, device=dev, generator=g) * 0.03 + 0.01).half(),
                     (torch.rand(B, 1, S, device=dev, generator=g) * 0.03 + 0.01).half()))
    q = torch.randn(B, 8, 64, device=dev, generator=g).bfloat16()
    n = np.random.default_rng(0).integers(64, 1025, size=B)
    pos, starts = torch.from_numpy(n - 1).to(dev), torch.zeros(B, dtype=torch.long, device=dev)
    byts = _attn_bytes(n - 1, np.zeros(B, np.int64), 0, B)
    f = lambda s: decode_attention(q, s[0], s[1], pos, starts, 0.14125, k_scale=s[2], v_scale=s[3])
    for i in range(args.warmup):
        f(sets[i % nsets])
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr):
        for s in sets:
            f(s)
    torch.cuda.synchronize()
    reps = max(1, args.steps // nsets)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        gr.replay()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (reps * nsets)
    gbs = byts / us / 1e3
    print(json.dumps({"metric": "decode attention GB/s, 256 x [64,1024] int8 KV", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
                      "steps": reps * nsets, "warmup": args.warmup, "ms_per_step": round(us / 1e3, 5), "higher_is_better": True,
                      "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": "C2 single-layer ragged int8-KV decode attention, cold (32 rotating cache sets)"},
                      "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None}}))


def bench_attn_ceiling(args):
    """Where the decode-attention kernel's time goes at the rollout's launch shape (2000 rows, 8 heads on 1 kv head, int8 KV,
    bf16 q, post epilogue): rows of n keys each, n swept from 1 to 1024, over 16 rotating cache sets (more bytes than the
    last-level cache holds, as in a real step), timed three ways - the kernel, its memory stream without its arithmetic
    and its arithmetic without the stream (uvmi_decode_attn_probe).  Prints the table and the line fitted through the
    stream-only times: a fixed cost per launch plus bytes at a marginal rate."""
    import ctypes as C
    from ultraviolet_amd import _lib as L
    from ultraviolet_amd.kernels.decode_attn import build_attn_args
    lib = L.lib()
    dev = "cuda:0"
    B, S, nsets = 2000, 1056, 16
    g = torch.Generator(device=dev).manual_seed(0)
    sets = [(torch.randint(-127, 128, (B, 1, S, 64), device=dev, dtype=torch.int8, generator=g),
             torch.randint(-127, 128, (B, 1, S, 64), device=dev, dtype=torch.int8, generator=g),
             (torch.rand(B, 1, S, device=dev, generator=g) * 0.03 + 0.01).half(),
             (torch.rand(B, 1, S, device=dev, generator=g) * 0.03 + 0.01).half()) for _ in range(nsets)]
    q = torch.randn(B, 8, 64, device=dev, generator=g).bfloat16()
    out = torch.empty_like(q)
    vhat = torch.nn.functional.normalize(torch.randn(B, 1, 64, device=dev, generator=g), dim=-1).contiguous()
    gate = torch.rand(B, 8, device=dev, generator=g) + 0.5
    xsa = torch.full((8,), 0.3, device=dev)
    starts = torch.zeros(B, dtype=torch.long, device=dev)
    rows = torch.arange(B, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    scratch = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    reps = max(2, args.steps // nsets) if args.steps > 0 else 4
    table = []
    for n in (1, 64, 128, 192, 256, 512, 1024):
        pos = torch.full((B,), n - 1, dtype=torch.long, device=dev)
        built = [build_attn_args(q, s[0], s[1], pos, starts, 0.14125, 0, False, s[2], s[3], 1, out, 0, rows, (vhat, gate, xsa, out.dtype))
                 for s in sets]
        byts = _attn_bytes(np.full(B, n - 1), np.zeros(B, np.int64), 0, B)
        us = {}
        for mode in (0, 1, 2):
            def run():
                for a, _ in built:
                    rc = lib.uvmi_decode_attn_probe(C.byref(a), mode, stream) if mode else lib.uvmi_decode_attn(C.byref(a), stream)
                    if rc:
                        L.check(rc, "uvmi_decode_attn")
            run()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            scratch.zero_()
            e0.record()
            for _ in range(reps):
                run()
            e1.record()
            torch.cuda.synchronize()
            us[mode] = e0.elapsed_time(e1) * 1e3 / (reps * nsets)
        table.append({"keys_per_row": n, "bytes_per_launch": int(byts), "kernel_us": round(us[0], 2), "stream_only_us": round(us[1], 2),
                      "arithmetic_only_us": round(us[2], 2), "kernel_GBs": round(byts / us[0] / 1e3, 1),
                      "stream_only_GBs": round(byts / us[1] / 1e3, 1)})
    x = np.array([t["bytes_per_launch"] for t in table], float)
    y = np.array([t["stream_only_us"] for t in table], float)
    slope, icpt = np.polyfit(x, y, 1)
    yk = np.array([t["kernel_us"] for t in table], float)
    slope_k, icpt_k = np.polyfit(x, yk, 1)
    at = 50.8e6
    print(json.dumps({"metric": "decode attention launch time by row length (kernel / stream only / arithmetic only)", "value": round(1e-3 / slope, 1),
                      "unit": "GB/s", "n_gpus": 1, "steps": reps * nsets, "warmup": 1, "ms_per_step": None, "higher_is_better": True,
                      "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": "decode attention, 2000 rows x n keys (n = 1 .. 1024), int8 KV, 16 rotating cache sets"},
                      "table": table,
                      "fit": {"stream_only": {"fixed_us": round(icpt, 2), "marginal_GBs": round(1e-3 / slope, 1)},
                              "kernel": {"fixed_us": round(icpt_k, 2), "marginal_GBs": round(1e-3 / slope_k, 1)},
                              "at_50.8_MB": {"stream_only_us": round(icpt + slope * at, 2), "kernel_us": round(icpt_k + slope_k * at, 2),
                                             "frac_if_only_the_stream_remained": round(at / (icpt + slope * at) / 1e3 / HBM_PEAK_GBS, 4)}}}))


def bench_gemm(args):
    """The projections of UV-50M as single launches, back to back in a graph on four rotating weight copies: this library's
    GEMM forms (config 0 = what the dispatcher picks for the shape; 4 / 3 = 64 x 64 / 128 x 128 tiles staged through registers;
    6 / 5 = 128 x 128 / 256 x 256 tiles loaded straight into LDS; 1 = the skinny form) beside the vendor library's (torch.mm /
    addmm, without the norm or SwiGLU launch it needs around it), at a full decode step's 2048 rows and a mixed pass's 33 216."""
    from ultraviolet_amd.kernels.gemm import RESID, STORE, SWIGLU, gemm_tn, interleave_gate_up
    dev, dt = "cuda:0", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    shapes = [("qkv+gates, pre-norm", 656, 640, STORE, True), ("o, residual update", 640, 512, RESID, False),
              ("gate-up, pre-norm + SwiGLU", 3328, 640, SWIGLU, True), ("down, residual update", 640, 1664, RESID, False),
              ("head", 32768, 640, STORE, False)]

    def timeit(fs, reps=4):
        for f in fs:
            f()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            for _ in range(reps):
                for f in fs:
                    f()
        gr.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        gr.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (reps * len(fs))

    table = []
    for M in (2048, 33216):
        for name, N, K, epi, norm in shapes:
            if name == "head" and M > 2048:
                continue
            ws = [(torch.randn(N, K, device=dev, generator=g) / K ** 0.5).to(dt) for _ in range(4)]
            a = torch.randn(M, K, device=dev, generator=g).to(dt)
            n_out = N // 2 if epi == SWIGLU else N
            out = torch.empty(M, n_out, device=dev, dtype=dt)
            x = torch.randn(M, N, device=dev, generator=g).to(dt) if epi == RESID else None
            row = {"rows": M, "projection": name, "N": N, "K": K, "GFLOP": round(2e-9 * M * N * K, 2)}
            timeit([(lambda w: (lambda: torch.mm(a, w.t())))(w) for w in ws])   # (the first graph on new buffers runs ~7 % slow)
            for cfg in (0, 1, 4, 3, 6, 5):
                kw = dict(epilogue=epi, norm_eps=1e-6 if norm else None, config=cfg)
                if epi == RESID:
                    kw.update(resid=x, ca=0.9, cb=1.1)
                tgt = x if epi == RESID else out
                try:
                    gemm_tn(a, ws[0], tgt, **kw)
                    torch.cuda.synchronize()
                except Exception:
                    continue
                row[f"config{cfg}_us"] = round(timeit([(lambda w: (lambda: gemm_tn(a, w, tgt, **kw)))(w) for w in ws]), 2)
            if epi == RESID:
                lib = [(lambda w: (lambda: torch.addmm(x, a, w.t(), beta=0.9, alpha=1.1, out=x)))(w) for w in ws]
            else:
                full = torch.empty(M, N, device=dev, dtype=dt)
                lib = [(lambda w: (lambda: torch.mm(a, w.t(), out=full)))(w) for w in ws]
            row["vendor_us"] = round(timeit(lib), 2)
            best = min(v for k, v in row.items() if k.endswith("_us") and k.startswith("config"))
            row["config0_PFLOPs"] = round(row["GFLOP"] / row["config0_us"], 3)
            row["best_own_us"] = best
            table.append(row)
    print(json.dumps({"metric": "projection GEMM launch time, UV-50M shapes", "value": None, "unit": "us", "n_gpus": 1, "steps": 16, "warmup": 1,
                      "ms_per_step": None, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": "UV-50M projections at 2048 and 33 216 rows, one launch each, four rotating weight copies"},
                      "table": table}))


def bench_c4(args):
    """BASELINE configs[3]: mixed batch, 64 prompt chunks x 512 tokens + 448 decode rows, one forward pass per iteration."""
    from ultraviolet_amd.engine import KVState, UVEngine, UVWeights, make_config
    from ultraviolet_amd.kernels.varlen_attn import packed_attention
    dev = "cuda:0"
    cfg = make_config("uv-50m-alpha")
    eng = UVEngine(UVWeights.random(cfg, seed=0, dtype=torch.bfloat16, device=dev, perturb=0.02), max_tokens=64 * 512 + 512)
    rng = np.random.default_rng(0)
    gen = torch.Generator(device=dev).manual_seed(0)
    st = KVState(cfg, 512, 2048 + 64, dev)
    nd, npf = 448, 64
    rows_d = torch.arange(nd, device=dev)
    ctx = torch.from_numpy(rng.integers(256, 2049, size=nd)).to(dev)
    _fill_cache(st, rows_d, ctx, gen)
    prompts = [rng.integers(1, cfg.vocab_size, size=512).tolist() for _ in range(npf)]
    pk = eng.pack_prompts(prompts, list(range(nd, nd + npf)), st.max_len, left_pad=False)
    tok_d = torch.from_numpy(rng.integers(1, cfg.vocab_size, size=nd)).to(dev)
    pos_d, starts_d = ctx.clone(), torch.zeros(nd, dtype=torch.long, device=dev)
    it = args.steps if args.steps > 0 else 100
    for _ in range(max(args.warmup, 2)):
        eng.mixed_step(pk, tok_d, pos_d, starts_d, rows_d, st)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(it):
        eng.mixed_step(pk, tok_d, pos_d, starts_d, rows_d, st)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = e0.elapsed_time(e1) / it
    # the two attention kernels alone, on the last pass's buffers
    N = pk["N"]
    b = eng.buf
    phases = {}
    for name, w in (("prefill_attn_global_us", 0), ("prefill_attn_local_us", cfg.window)):
        out = torch.empty_like(b["q"][:N])
        for _ in range(3):
            packed_attention(b["q"][:N], b["k"][:N], b["v"][:N], pk["cu"], cfg.attn_scale, w, out=out, workspace=eng.pf_ws)
        e0.record()
        for _ in range(20):
            packed_attention(b["q"][:N], b["k"][:N], b["v"][:N], pk["cu"], cfg.attn_scale, w, out=out, workspace=eng.pf_ws)
        e1.record()
        torch.cuda.synchronize()
        phases[name] = round(e0.elapsed_time(e1) * 1e3 / 20, 1)
    # the backward of the same packed attention (the trainer side's first kernel): output gradient -> dq, dk, dv
    from ultraviolet_amd.kernels.varlen_attn import packed_attention_backward
    go = torch.randn(N, cfg.n_heads, cfg.head_dim, device=dev, generator=gen).to(torch.bfloat16)
    qc, kc, vc = (b[n_][:N].contiguous() for n_ in ("q", "k", "v"))
    for name, w in (("prefill_attn_bwd_global_us", 0), ("prefill_attn_bwd_local_us", cfg.window)):
        o = packed_attention(qc, kc, vc, pk["cu"], cfg.attn_scale, w)
        for _ in range(3):
            packed_attention_backward(go, qc, kc, vc, o, pk["cu"], cfg.attn_scale, w)
        e0.record()
        for _ in range(10):
            packed_attention_backward(go, qc, kc, vc, o, pk["cu"], cfg.attn_scale, w)
        e1.record()
        torch.cuda.synchronize()
        phases[name] = round(e0.elapsed_time(e1) * 1e3 / 10, 1)
    fl_g = 4 * 8 * 64 * npf * (512 * 513 // 2)
    fl_l = 4 * 8 * 64 * npf * (512 * 256 - 256 * 255 // 2)
    ntok = N + nd
    print(json.dumps({"metric": "mixed-batch forward tok/s (64 x 512 prefill + 448 decode rows)", "value": round(ntok / (ms / 1e3), 1),
                      "unit": "tok/s", "n_gpus": 1, "steps": it, "warmup": max(args.warmup, 2), "ms_per_step": round(ms, 4),
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": "C4 mixed batch: 64 prompt chunks x 512 tokens (causal, window 256 on local layers, int8 append "
                                             "fused) packed with 448 decode rows, contexts U{256..2048}; one forward pass per step, eager launches",
                                 "token_rows": ntok, "wall_ms_per_step": round(wall * 1e3 / it, 4), **phases,
                                 "prefill_attn_global_TFLOPs": round(fl_g / phases["prefill_attn_global_us"] / 1e6, 1),
                                 "prefill_attn_local_TFLOPs": round(fl_l / phases["prefill_attn_local_us"] / 1e6, 1),
                                 "prefill_attn_bwd_global_TFLOPs": round(2.5 * fl_g / phases["prefill_attn_bwd_global_us"] / 1e6, 1),
                                 "prefill_attn_bwd_local_TFLOPs": round(2.5 * fl_l / phases["prefill_attn_bwd_local_us"] / 1e6, 1)}}))


def bench_c3(args):
    """BASELINE configs[2]: 512 slots, contexts U{128..2048}, retire p = 0.01 per step, 64-token prompts admitted into freed
    slots inside decode passes; 256 steps."""
    from ultraviolet_amd.engine import UVEngine, UVWeights, make_config
    from ultraviolet_amd.engine.rollout import Rollout
    dev = "cuda:0"
    cfg = make_config("uv-50m-alpha")
    eng = UVEngine(UVWeights.random(cfg, seed=0, dtype=torch.bfloat16, device=dev, perturb=0.02), max_tokens=2048)
    B = 512
    K = args.steps if args.steps > 0 else 256
    W = args.warmup
    g = c3_rollout(eng, cfg, B, W + K, device_admit=not args.host_admit)
    g.precapture()

    def run(n):
        s0 = g.n_decode_steps
        while g.n_decode_steps - s0 < n:
            g.chunk()
        if g.harvest_pending:   # (chunk() leaves its harvest for the next call to take)
            g.harvest_end()

    def generated():
        return int(g.slot_cnt[g.slot_req >= 0].sum()) + g.n_tokens

    run(W)
    torch.cuda.synchronize()
    tok0, s0, m0 = generated(), g.n_decode_steps, g.n_mixed_steps
    t0 = time.perf_counter()
    run(K)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    steps = g.n_decode_steps - s0
    gen_tok = generated() - tok0
    print(json.dumps({"metric": "decode tok/s, 512 slots with churn (retire p=0.01, 64-token prompts admitted in mixed batches)",
                      "value": round(gen_tok / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": W,
                      "ms_per_step": round(dt * 1e3 / steps, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                      "dtype": "bf16", "data": "synthetic",
                      "config": {"workload": "C3 continuous batching: UV-50M bf16, int8 KV, 512 slots, contexts U{128..2048} materialised in the "
                                             "cache, Bernoulli(0.01) retirement per slot and step on the device, 64-token prompts admitted into "
                                             "freed slots inside decode passes, harvest every 4 steps (its results taken one step later)",
                                 "tokens_timed": gen_tok, "mixed_steps": g.n_mixed_steps - m0, "requests_finished": g.next_req - len(g.meta),
                                 "active_at_end": g.n_active(), "mean_active_slots": round(gen_tok / steps, 1),
                                 "admission": "host: free list and queue in Python" if args.host_admit else
                                              "device: uvmi_sched_plan_admit takes staged prompts and reusable slots itself",
                                 "full_slot_tok_per_s": round(B * steps / dt, 1)}}))


def bench_copy(args):
    """Plain device-to-device copy of a known size: the calibration kernel for the FETCH_SIZE / WRITE_SIZE counters."""
    n = 1 << 30
    a = torch.empty(n, dtype=torch.uint8, device="cuda:0").fill_(1)
    b = torch.empty_like(a)
    for _ in range(max(args.warmup, 1)):
        b.copy_(a)
    torch.cuda.synchronize()
    reps = args.steps if args.steps > 0 else 10
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        b.copy_(a)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / reps
    print(json.dumps({"metric": "device copy GB/s (read + write)", "value": round(2 * n / us / 1e3, 1), "unit": "GB/s", "n_gpus": 1,
                      "steps": reps, "warmup": args.warmup, "ms_per_step": round(us / 1e3, 4), "higher_is_better": True, "scaling": "weak",
                      "vs_baseline": None, "dtype": "u8", "data": "synthetic",
                      "config": {"workload": "copy of 1 GiB (counter calibration): reads 1073741824 B, writes 1073741824 B per launch"}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0, help="timed decode steps (0: the whole rollout after warm-up)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--workload", default="c5", choices=["c5", "c2", "c3", "c4", "copy", "attn-ceiling", "gemm"])
    ap.add_argument("--host-admit", action="store_true", help="c3: the host chooses the slots of admitted prompts (default: the device does)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (rollouts shard by sequence with no communication between ranks); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    if args.workload == "copy":
        bench_copy(args)
    elif args.workload == "c2":
        if args.steps <= 0:
            args.steps = 3200
        bench_c2(args)
    elif args.workload == "c3":
        bench_c3(args)
    elif args.workload == "c4":
        bench_c4(args)
    elif args.workload == "attn-ceiling":
        bench_attn_ceiling(args)
    elif args.workload == "gemm":
        bench_gemm(args)
    else:
        bench_c5(args)


if __name__ == "__main__":
    main()
