"""Continuous-batching rollout driver on the device-side slot table.

Mirrors the reference's StreamGen (scripts/rl_stream.py:39-154: add / chunk / n_active / n_outstanding / drop_queued,
results as (meta, tokens, behaviour log-probs, start_version)) and generate_continuous (ultraviolet/model.py:1266-1354),
with the per-step bookkeeping moved to the GPU:

  * the slot table (request id, count, limit, current token, position, output rows) lives in HBM (csrc/sched.hip);
  * each decode step is compact -> trunk over the active rows only -> head GEMM -> fused sampler -> commit, captured
    once per bucket of active-row counts and replayed; no step reads anything back to the host;
  * the host only polls a completion ring every `check_every` steps (one small copy), harvests finished rows and
    prefills queued requests into the freed slots.

Sampling is keyed by (seed, request id, token index), so a request's tokens do not depend on the slot it lands in or on
when it is admitted; the reference's torch.rand stream (perf.py:595) has no such property."""
from __future__ import annotations

import collections
import ctypes as C

import numpy as np
import torch

from .. import _lib as L
from ..kernels.fused_sample import fused_sample_seeded, greedy_sample
from .model import KVState, UVEngine


class Rollout:
    def __init__(self, engine: UVEngine, slots: int, max_prompt: int, max_new: int, temperature: float = 1.0,
                 seed: int = 0, eos_id: int | None = None, check_every: int = 16, bucket: int = 128,
                 use_graph: bool = True, retire_p: float = 0.0, left_pad: bool = False, mixed: bool = False,
                 admit_cap: int = 16, top_k: int = 0, top_p: float = 1.0, kv_dtype: str = "int8", overlap_harvest: bool = False,
                 share_prompts: bool = False, device_admit: bool = False):
        self.e, self.cfg = engine, engine.cfg
        self.top_k, self.top_p = int(top_k), float(top_p)   # truncated sampling (sample(), model.py:1200-1209); off by default
        self.B, self.max_prompt, self.max_new = slots, max_prompt, max_new
        self.T, self.seed, self.eos = float(temperature), int(seed), eos_id
        self.ce, self.bucket, self.use_graph = check_every, bucket, use_graph
        self.retire_p, self.left_pad = float(retire_p), left_pad
        self.mixed = mixed                        # admit while decoding: prompts ride in the same pass as the decode rows
        self.device_admit = bool(device_admit)    # the free-slot choice and the FIFO queue of a mixed step live on the device
        assert not device_admit or mixed, "device_admit plans the admissions of mixed steps: it needs mixed=True"
        self.n_mixed_steps = 0
        dev = engine.device
        self.dev = dev
        assert slots <= engine.max_tokens
        self.st = KVState(self.cfg, slots, max_prompt + max_new + 1, dev, kv_dtype=kv_dtype, dtype=engine.dtype)
        z = lambda *s, dt=torch.long: torch.zeros(*s, dtype=dt, device=dev)
        self.slot_req = torch.full((slots,), -1, dtype=torch.long, device=dev)
        self.slot_cnt, self.slot_limit, self.slot_tok = z(slots), z(slots), z(slots)
        self.out_tok = z(slots, max_new, dt=torch.int32)
        self.out_lp = z(slots, max_new, dt=torch.float32)
        self.done_cap = 2 * slots
        self.done_req, self.done_slot, self.done_cnt = z(self.done_cap), z(self.done_cap), z(self.done_cap)
        self.counters = z(4, dt=torch.int32)
        s = L.SchedState()
        s.slot_req, s.slot_cnt, s.slot_limit, s.slot_tok = (t.data_ptr() for t in (self.slot_req, self.slot_cnt, self.slot_limit, self.slot_tok))
        s.pos, s.starts = self.st.pos.data_ptr(), self.st.starts.data_ptr()
        s.out_tok, s.out_lp = self.out_tok.data_ptr(), self.out_lp.data_ptr()
        s.done_req, s.done_slot, s.done_cnt, s.counters = (t.data_ptr() for t in (self.done_req, self.done_slot, self.done_cnt, self.counters))
        s.max_new, s.eos_id, s.B, s.done_cap = max_new, -1 if eos_id is None else int(eos_id), slots, self.done_cap
        self.sched = s
        # Per-token arrays of a step: Np packed tokens of the prompts admitted with the step (mixed batches only), then
        # the decode rows of the bucket (bucket length <= slots).  The decode views are what the compaction kernel fills.
        self.A = int(admit_cap) if mixed else 0                     # prompts one mixed step can admit
        self.Np = (self.A * max_prompt + 15) // 16 * 16             # packed prompt tokens of a mixed step
        A, Np = self.A, self.Np
        assert not mixed or Np + slots <= engine.max_tokens, "engine.max_tokens too small for admit_cap * max_prompt + slots"
        self.tok_all, self.pos_all, self.row_all, self.last_all = (z(Np + slots) for _ in range(4))
        self.req_all, self.cnt_all = z(A + slots), z(A + slots)
        self.act, self.tok_c, self.pos_c = self.row_all[Np:], self.tok_all[Np:], self.pos_all[Np:]
        self.req_c, self.cnt_c = self.req_all[A:], self.cnt_all[A:]
        self.starts_c = z(slots)
        self._commit_args = L.SampleCommit(C.pointer(self.sched), self.act.data_ptr(), self.tok_c.data_ptr(), self.pos_c.data_ptr(),
                                           self.starts_c.data_ptr(), self.req_c.data_ptr(), self.cnt_c.data_ptr(), self.retire_p,
                                           self.seed & (2 ** 64 - 1))
        if mixed:
            # admission staging, one host -> device copy per mixed step: [tokens Np | cu A+1 | slot A | start A | limit A | req A]
            self.stage_n = Np + (A + 1) + 3 * A
            self.stage_h = torch.zeros(self.stage_n + A, dtype=torch.long, pin_memory=True)
            self.stage_d = z(self.stage_n)
            o = Np
            self.adm_cu, o = self.stage_d[o:o + A + 1], o + A + 1
            self.adm_slot, o = self.stage_d[o:o + A], o + A
            self.adm_start, o = self.stage_d[o:o + A], o + A
            self.adm_limit, o = self.stage_d[o:o + A], o + A
            self.gather_idx = torch.cat([z(A), Np + torch.arange(slots, device=dev)])   # rows of the hidden that get sampled
            self.adm_slot.fill_(-1)
            self._stage_ev = torch.cuda.Event()
        if self.device_admit:
            # the admission queue: a ring of staged prompts [length, request id, limit, tokens ...] the planning kernel takes
            # from; the host only appends rows (and the staged count after them) and learns what was admitted from the harvest
            self.q_cap = 1 << max(6, (4 * A - 1).bit_length())
            self.q_stride = max_prompt + 3
            self.q_buf, self.q_ctl = z(self.q_cap, self.q_stride), z(4)
            self.q_rows_h = torch.zeros(self.q_cap, self.q_stride, dtype=torch.long, pin_memory=True)
            self.q_ctl_h = torch.zeros(1, dtype=torch.long, pin_memory=True)
            self.slot_hold = z(slots, dt=torch.int32)
            s.slot_hold, s.q_buf, s.q_ctl, s.q_cap, s.q_stride = self.slot_hold.data_ptr(), self.q_buf.data_ptr(), self.q_ctl.data_ptr(), self.q_cap, self.q_stride
            self.q_tail = 0                           # prompts staged so far
            self.q_head = 0                           # prompts the device is known to have admitted (as of the last harvest)
            self.staged = collections.deque()         # (request id, meta) of staged prompts not yet known to be admitted
            self.n_free_dev = slots                   # reusable slots as of the last harvest, minus what may have been admitted since
            self._q_ev = torch.cuda.Event()
        # harvest staging: a launch packs up to hv_rows new completion records and their output rows; the host takes the header
        # and then exactly the finished tokens, through pinned buffers (no indexing launches, no pageable copies)
        self.hv_rows = min(slots, 128)
        self.hv_hdr, self.hv_tok, self.hv_lp = z(8 + 4 * self.hv_rows), z(self.hv_rows * max_new, dt=torch.int32), z(self.hv_rows * max_new, dt=torch.float32)
        self.hv_hdr_h, self.hv_tok_h, self.hv_lp_h = (torch.zeros(t.shape, dtype=t.dtype, pin_memory=True) for t in (self.hv_hdr, self.hv_tok, self.hv_lp))
        self._hv_ev, self._hv_ev2 = torch.cuda.Event(), torch.cuda.Event()
        self._hv_stream = torch.cuda.Stream(device=dev)   # default priority; carries only the harvest's device -> host copies
        self.harvest_pending = False
        self.overlap_harvest = bool(overlap_harvest)
        self.share_prompts = bool(share_prompts)   # admission prefills identical prompts of a call once and copies their cache rows
        self.graphs: dict[int, torch.cuda.CUDAGraph] = {}
        self.mixed_graphs: dict[int, torch.cuda.CUDAGraph] = {}
        self.queue = collections.deque()
        self.meta: dict[int, tuple] = {}          # request id -> (meta, start_version)
        self.free = list(range(slots))[::-1]
        self.next_req = 0
        self.n_active_host = 0                    # upper bound on active slots (exact after each poll / admit)
        self.done_seen = 0
        self._dense_n = None                      # bucket the dense step arrays are valid for (None: stale, compact first)
        self.version = 0                          # advanced by the caller after each weight update (scripts/rl_grpo.py:1309)
        self._admit_version = 0                   # version at the launch of the last step that admitted on the device
        self._scalar_epoch = getattr(self.e.w, "scalar_epoch", 0)
        self.n_decode_steps = 0
        self.n_tokens = 0
        self.n_prefill_tokens = 0                 # prompt tokens that went through a prefill pass of _admit (shared prompts once)

    # ------------------------------------------------------------------------------------------------ requests
    def add(self, prompt_ids, meta, limit: int | None = None):
        assert 0 < len(prompt_ids) <= self.max_prompt, "prompt longer than max_prompt"
        ids = list(prompt_ids)
        self.queue.append((ids, meta, self.max_new if limit is None else min(int(limit), self.max_new), np.asarray(ids, dtype=np.int64)))

    def n_active(self) -> int:
        if self.device_admit:
            return self.n_active_host      # an upper bound between harvests, exact after one
        return self.B - len(self.free)

    def n_outstanding(self) -> int:
        if self.device_admit:
            return len(self.queue) + len(self.meta)
        return len(self.queue) + self.n_active()

    def drop_queued(self, pred) -> int:
        """Drop the queued requests whose meta satisfies pred (prompts already staged on the device stay)."""
        keep = [x for x in self.queue if not pred(x[1])]
        n = len(self.queue) - len(keep)
        self.queue = collections.deque(keep)
        return n

    @torch.no_grad()
    def sync_weights_inplace(self, params: dict):
        """New policy weights for the following steps (reference: sync_weights_inplace, scripts/rl_stream.py:22-36): the
        fused tensors are overwritten in place, so captured step graphs stay valid; they are only dropped when a residual
        scalar (a launch argument) changed.  `version` is the caller's to advance, as in the reference's loop
        (scripts/rl_grpo.py:1308-1309: sync_weights_inplace(gen_m, raw); gen.version += 1); requests admitted after that
        carry the new value as their start_version."""
        self.e.w.load_(params)
        self._check_weight_epoch()
        torch.cuda.synchronize(self.dev)

    def _check_weight_epoch(self):
        """Drop the captured graphs when the engine's weights were reloaded with different launch-argument scalars since the
        graphs were captured - whoever reloaded them (this object, a patched model's refresh, perf.sync_weights_inplace)."""
        ep = getattr(self.e.w, "scalar_epoch", 0)
        if ep != self._scalar_epoch:
            self._scalar_epoch = ep
            self.graphs.clear()
            self.mixed_graphs.clear()

    # ------------------------------------------------------------------------------------------------ admission
    @torch.no_grad()
    def _admit(self):
        """Prefill queued requests into free slots (FIFO), in calls of at most engine.max_tokens packed tokens."""
        e = self.e
        while self.queue and self.free:
            # prompts that occur several times in the call (a sampling group) are prefilled once: only their first occurrence
            # counts against the pass's token budget
            batch, ntok, first, src = [], 0, {}, []
            while self.queue and len(batch) < len(self.free):
                it = self.queue[0]
                key = it[3].tobytes() if self.share_prompts else None
                new = key is None or key not in first
                if new and ntok + len(it[0]) > e.max_tokens:
                    break
                self.queue.popleft()
                if key is not None:
                    src.append(first.setdefault(key, len(batch)))
                if new:
                    ntok += len(it[0])
                batch.append(it)
            if not batch:
                raise RuntimeError("a queued prompt exceeds the engine's max_tokens")
            slots = [self.free.pop() for _ in batch]
            reqs = list(range(self.next_req, self.next_req + len(batch)))
            self.next_req += len(batch)
            self.n_prefill_tokens += ntok
            if len(first) < len(batch) and self.share_prompts:
                uniq = sorted(first.values())
                at = {j: u for u, j in enumerate(uniq)}
                h = e.prefill([batch[j][3] for j in uniq], [slots[j] for j in uniq], self.st, left_pad=self.left_pad)
                dup = [j for j in range(len(batch)) if src[j] != j]
                ix = torch.as_tensor([[at[s_] for s_ in src], [slots[s_] for s_ in src], slots], dtype=torch.long).to(self.dev)
                d_ix = torch.as_tensor(dup, dtype=torch.long).to(self.dev)
                self.st.copy_rows(ix[1][d_ix], ix[2][d_ix], max(len(batch[j][3]) for j in uniq))
                h = h.index_select(0, ix[0])
            else:
                h = e.prefill([b[3] for b in batch], slots, self.st, left_pad=self.left_pad)
            x = e.head(h)
            # request ids, slots and limits in one host -> device copy (named: they must outlive the launch call)
            req_t, slot_t, lim_t = torch.as_tensor([reqs, slots, [b[2] for b in batch]], dtype=torch.long).to(self.dev).unbind(0)
            tok, lp = self._sample(x, req_t, torch.zeros_like(req_t))
            rc = L.lib().uvmi_sched_admit(C.byref(self.sched), len(batch), slot_t.data_ptr(), req_t.data_ptr(), lim_t.data_ptr(),
                                          tok.data_ptr(), lp.data_ptr(), L.stream_ptr(tok))
            L.check(rc, "uvmi_sched_admit")
            for r, b in zip(reqs, batch):
                self.meta[r] = (b[1], self.version)
            self.n_active_host += len(batch)
            self._dense_n = None

    def _sample(self, x, req, cnt, commit=None):
        if self.T > 0:
            return fused_sample_seeded(x, self.seed, req, cnt, self.cfg.softcap, self.T, top_k=self.top_k, top_p=self.top_p, commit=commit)
        return greedy_sample(x, self.cfg.softcap, commit=commit)

    @torch.no_grad()
    def _admit_mixed(self) -> bool:
        """Admission fused with a decode step: queued prompts (FIFO; at most admit_cap prompts and Np tokens) are prefilled
        in the same forward pass that decodes the active slots; one head GEMM and one sampler launch cover the prompts'
        first tokens and the decode rows.  The host only chooses the slots and uploads the packed prompt tokens with their
        cu_seqlens (one copy); positions, cache rows and the slot table entries are built on the device, so the whole
        step is one graph replay.  Returns False when nothing fits."""
        n = self.bucket_for(self.n_active_host)
        A, Np = self.A, self.Np
        batch, ntok = [], 0
        while self.queue and len(batch) < min(len(self.free), A) and ntok + len(self.queue[0][0]) <= Np:
            it = self.queue.popleft()
            batch.append(it)
            ntok += len(it[0])
        if not batch:
            return False
        na = len(batch)
        slots = [self.free.pop() for _ in batch]
        reqs = list(range(self.next_req, self.next_req + na))
        self.next_req += na
        lens = np.fromiter((len(b[0]) for b in batch), dtype=np.int64, count=na)
        starts = (int(lens.max()) - lens) if self.left_pad else np.zeros(na, np.int64)
        self._stage_ev.synchronize()                        # the previous upload has left the pinned buffer
        h = self.stage_h.numpy()
        h[:] = 0
        h[:ntok] = np.concatenate([b[3] for b in batch])
        o = Np
        h[o] = 0
        h[o + 1:o + 1 + na] = np.cumsum(lens)
        h[o + 1 + na:o + 1 + A] = ntok
        o += A + 1
        h[o:o + A] = -1
        h[o:o + na] = slots
        o += A
        h[o:o + na] = starts
        o += A
        h[o:o + na] = [b[2] for b in batch]
        o += A
        h[o:o + na] = reqs                                  # request ids ride behind the staged block
        self.stage_d.copy_(self.stage_h[:self.stage_n], non_blocking=True)
        self.tok_all[:Np].copy_(self.stage_d[:Np])
        self.req_all[:A].copy_(self.stage_h[self.stage_n:], non_blocking=True)
        self._stage_ev.record()
        if self.use_graph:
            (self.mixed_graphs.get(n) or self._capture(n, mixed=True)).replay()
        else:
            self._mixed_body(n)
        for r, b in zip(reqs, batch):
            self.meta[r] = (b[1], self.version)
        self.n_active_host += na
        self._dense_n = None                                # the step's dense arrays predate the admission
        self.n_decode_steps += 1
        self.n_mixed_steps += 1
        return True

    # ---- device-side admission: the host stages prompts and launches; the slot choice and the queue are the device's
    @torch.no_grad()
    def _stage_prompts(self):
        """Append queued prompts to the device ring while it has room (room is counted against the admissions the host has
        seen, a lower bound of the device's), then publish the staged count.  Request ids are assigned here, in arrival
        order.  Copies are stream-ordered ahead of the next step's planning kernel."""
        room = self.q_cap - (self.q_tail - self.q_head)
        k = min(room, len(self.queue))
        if k <= 0:
            return
        self._q_ev.synchronize()                            # the previous upload has left the pinned rows
        rows = self.q_rows_h.numpy()
        first = self.q_tail % self.q_cap
        for j in range(k):
            ids, meta, limit, arr = self.queue.popleft()
            r = rows[(first + j) % self.q_cap]
            r[0], r[1], r[2] = len(ids), self.next_req, limit
            r[3:3 + len(ids)] = arr
            self.meta[self.next_req] = (meta, None)         # start_version is set when the admission is seen
            self.staged.append(self.next_req)
            self.next_req += 1
        n1 = min(k, self.q_cap - first)
        self.q_buf[first:first + n1].copy_(self.q_rows_h[first:first + n1], non_blocking=True)
        if k > n1:
            self.q_buf[:k - n1].copy_(self.q_rows_h[:k - n1], non_blocking=True)
        self.q_tail += k
        self.q_ctl_h[0] = self.q_tail
        self.q_ctl[:1].copy_(self.q_ctl_h, non_blocking=True)
        self._q_ev.record()

    @torch.no_grad()
    def _admit_device(self) -> bool:
        """A decode step that also admits what the device finds admissible: one graph replay, nothing uploaded.  The host's
        part is the decision to launch it - it knows how many prompts are staged and, from the last harvest, how many slots
        were reusable - and an upper bound on the active slots for the bucket.  Returns False when there is nothing to admit."""
        pending = self.q_tail - self.q_head
        if pending <= 0 or self.n_free_dev <= 0:
            return False
        may = min(self.A, pending, self.n_free_dev)
        n = self.bucket_for(self.n_active_host)
        if self.use_graph:
            (self.mixed_graphs.get(n) or self._capture(n, mixed=True)).replay()
        else:
            self._mixed_body(n)
        self.n_active_host = min(self.B, self.n_active_host + may)   # upper bound until the next harvest tells
        self.n_free_dev -= may
        self._admit_version = self.version
        self._dense_n = None
        self.n_decode_steps += 1
        self.n_mixed_steps += 1
        return True

    def _mixed_body(self, n: int):
        """compact -> prompt tables -> one trunk pass over Np prompt tokens + n decode rows -> head -> sampler -> commit
        (decode rows) + admit (prompts).  Every launch has fixed shapes; what varies lives in device arrays."""
        e, lib, A, Np = self.e, L.lib(), self.A, self.Np
        sp = L.stream_ptr(self.act)
        if self.device_admit:   # compaction, admission plan and prompt tables in one launch
            L.check(lib.uvmi_sched_step_plan(C.byref(self.sched), n, self.act.data_ptr(), self.tok_c.data_ptr(), self.pos_c.data_ptr(),
                                             self.starts_c.data_ptr(), self.req_c.data_ptr(), self.cnt_c.data_ptr(), A, Np, int(self.left_pad),
                                             self.adm_cu.data_ptr(), self.adm_slot.data_ptr(), self.adm_start.data_ptr(),
                                             self.adm_limit.data_ptr(), self.req_all.data_ptr(), self.tok_all.data_ptr(),
                                             self.pos_all.data_ptr(), self.row_all.data_ptr(), self.last_all.data_ptr(),
                                             self.gather_idx.data_ptr(), self.last_all[Np:].data_ptr(), sp), "uvmi_sched_step_plan")
        else:
            L.check(lib.uvmi_sched_compact(C.byref(self.sched), n, self.act.data_ptr(), self.tok_c.data_ptr(), self.pos_c.data_ptr(),
                                           self.starts_c.data_ptr(), self.req_c.data_ptr(), self.cnt_c.data_ptr(), sp), "uvmi_sched_compact")
            L.check(lib.uvmi_sched_expand(C.byref(self.sched), A, Np, self.adm_cu.data_ptr(), self.adm_slot.data_ptr(), self.adm_start.data_ptr(),
                                          self.pos_all.data_ptr(), self.row_all.data_ptr(), self.last_all.data_ptr(), self.gather_idx.data_ptr(),
                                          sp), "uvmi_sched_expand")
            self.last_all[Np:Np + n].copy_(self.pos_all[Np:Np + n])
        h = e.mixed_trunk(self.tok_all, self.pos_all, self.row_all, self.last_all, Np, n, self.adm_cu, self.starts_c[:n], self.st)
        x = e.head(h.index_select(0, self.gather_idx[:A + n]))
        tok, lp = self._sample(x, self.req_all[:A + n], self.cnt_all[:A + n])
        # (the sampler's outputs are read in place: rows 0..A-1 are the prompts' first tokens, the rest the decode rows')
        tok_d, lp_d = tok[A:], lp[A:]
        L.check(lib.uvmi_sched_commit(C.byref(self.sched), n, self.act.data_ptr(), tok_d.data_ptr(), lp_d.data_ptr(),
                                      self.retire_p, self.seed & (2 ** 64 - 1), sp), "uvmi_sched_commit")
        L.check(lib.uvmi_sched_admit(C.byref(self.sched), A, self.adm_slot.data_ptr(), self.req_all.data_ptr(), self.adm_limit.data_ptr(),
                                     tok.data_ptr(), lp.data_ptr(), sp), "uvmi_sched_admit")

    # ------------------------------------------------------------------------------------------------ decode
    def _compact(self, n: int):
        """Dense arrays of the active slots for a bucket of n rows (active slots first, ascending)."""
        L.check(L.lib().uvmi_sched_compact(C.byref(self.sched), n, self.act.data_ptr(), self.tok_c.data_ptr(), self.pos_c.data_ptr(),
                                           self.starts_c.data_ptr(), self.req_c.data_ptr(), self.cnt_c.data_ptr(), L.stream_ptr(self.act)),
                "uvmi_sched_compact")
        self._dense_n = n

    def _step_body(self, n: int):
        """One decode step on the dense arrays of bucket n (compacted by the caller when they are stale: after an admission,
        or when the bucket changes); the commit carries them to the next step, so a step has no compaction launch."""
        e, st = self.e, self.st
        act, pos, starts = self.act[:n], self.pos_c[:n], self.starts_c[:n]

        def attn(l, q):
            return self._attention(l, q, st, pos, starts, n, act)

        fused = (lambda l: e.fused_cache_attention(l, self.tok_c[:n], st, pos, starts, n, rows=act)) if e.fuse_qkv else None
        h = e._trunk(self.tok_c[:n], pos, n, attn, rows=act, st=st, fused_attn=fused, defer_final_norm=True)
        x = e.head_of(h)
        # the sampler's launch also commits the rows' tokens (what uvmi_sched_commit_dense does in a launch of its own)
        self._sample(x, self.req_c[:n], self.cnt_c[:n], commit=self._commit_args)

    def _attention(self, l, q, st, pos, starts, n, act):
        return self.e.cache_attention(l, q, st, pos, starts, n, rows=act)

    def bucket_for(self, n_active: int) -> int:
        return min(self.B, max(self.bucket, -(-n_active // self.bucket) * self.bucket))

    def _capture(self, n: int, mixed: bool = False):
        """Capture the step for a bucket of n rows (mixed: the step that also admits prompts).  A captured step mutates the
        slot table, so the kernels and GEMM shapes are first warmed up on the live state, which is then restored; capture
        itself executes nothing."""
        body = self._mixed_body if mixed else self._step_body
        keep = [t.clone() for t in self._mutable()]
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            if not mixed:
                self._compact(n)   # (a bucket below the active count raises the overflow flag: restored with the rest)
            body(n)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        for t, k in zip(self._mutable(), keep):
            t.copy_(k)
        self._dense_n = None
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            body(n)
        (self.mixed_graphs if mixed else self.graphs)[n] = g
        return g

    @torch.no_grad()
    def precapture(self):
        """Capture every bucket from the current active count downwards (the count only shrinks between admissions), so
        that no capture happens inside a timed or latency-sensitive region."""
        if self.use_graph:
            for n in range(self.bucket, self.bucket_for(self.n_active_host) + 1, self.bucket):
                if n not in self.graphs:
                    self._capture(min(n, self.B))
                if self.mixed and (self.queue or (self.device_admit and self.q_tail > self.q_head)) and n not in self.mixed_graphs:
                    self._capture(min(n, self.B), mixed=True)

    @torch.no_grad()
    def step_inputs(self):
        """(n, slot, token, position, start) of the rows the next step() will run: views of the dense step arrays of its
        bucket of n rows (slot -1: padding).  step() overwrites them with the following step's."""
        n = self.bucket_for(self.n_active_host)
        if self._dense_n != n:
            self._compact(n)
        return n, self.act[:n], self.tok_c[:n], self.pos_c[:n], self.starts_c[:n]

    @torch.no_grad()
    def step(self):
        """One decode step for every active slot (graph replay of the bucket that covers the active count)."""
        n = self.bucket_for(self.n_active_host)
        g = (self.graphs.get(n) or self._capture(n)) if self.use_graph else None
        if self._dense_n != n:
            self._compact(n)
        if g is None:
            self._step_body(n)
        else:
            g.replay()
        self.n_decode_steps += 1

    def _mutable(self):
        """State a decode step writes.  The KV cache is left out on purpose: the warm-up step writes K/V at the current
        positions, and the real replay rewrites exactly those slots with identical inputs (as in model.py:1126-1127)."""
        m = [self.slot_req, self.slot_cnt, self.slot_limit, self.slot_tok, self.st.pos, self.st.starts, self.out_tok, self.out_lp,
             self.done_req, self.done_slot, self.done_cnt, self.counters, self.act, self.tok_c, self.pos_c, self.starts_c, self.req_c,
             self.cnt_c]
        return m + [self.q_ctl, self.slot_hold] if self.device_admit else m

    # ------------------------------------------------------------------------------------------------ harvest
    @torch.no_grad()
    def harvest_begin(self):
        """Enqueue the harvest: a launch packs the new completion records and their output rows, and the header starts
        its way to the host.  Nothing waits; harvest_end() takes the results.  Work enqueued in between (a decode step)
        runs while the host does so - it may not admit requests, since the rows of finished slots must stay untouched."""
        assert not self.harvest_pending
        rc = L.lib().uvmi_sched_harvest(C.byref(self.sched), self.done_seen, self.hv_rows, self.hv_hdr.data_ptr(), self.hv_tok.data_ptr(),
                                        self.hv_lp.data_ptr(), L.stream_ptr(self.hv_hdr))
        L.check(rc, "uvmi_sched_harvest")
        self.hv_hdr_h.copy_(self.hv_hdr, non_blocking=True)
        self._hv_ev.record()
        self.harvest_pending = True

    @torch.no_grad()
    def harvest_end(self):
        """Take the results of harvest_begin(): finished requests as (meta, tokens, logp float32 array, start_version);
        frees their slots.  The finished tokens come over on a second stream, so they do not queue behind a decode step
        enqueued since."""
        assert self.harvest_pending
        out = []
        while True:
            self._hv_ev.synchronize()
            self.harvest_pending = False
            hdr = self.hv_hdr_h.numpy()
            n_done, k = int(hdr[1]), int(hdr[3])
            if hdr[2]:
                raise RuntimeError("active slots exceeded the captured bucket (host bound on active slots was wrong)")
            assert n_done - self.done_seen <= self.done_cap, "completion ring overflow: poll more often"
            if k == 0:
                break
            rec = hdr[4:4 + 4 * k].reshape(k, 4)
            total = int(rec[-1, 3] + rec[-1, 2])
            if total:
                with torch.cuda.stream(self._hv_stream):   # (the packing launch has finished: its header has arrived)
                    self.hv_tok_h[:total].copy_(self.hv_tok[:total], non_blocking=True)
                    self.hv_lp_h[:total].copy_(self.hv_lp[:total], non_blocking=True)
                    self._hv_ev2.record()
                self._hv_ev2.synchronize()
            toks, lps = self.hv_tok_h.numpy(), self.hv_lp_h.numpy()
            self._see_admissions(hdr)
            # arrival order inside one step is not deterministic: sort by request
            for r, s_, c, o in rec[np.argsort(rec[:, 0], kind="stable")].tolist():
                meta, v0 = self.meta.pop(r)
                out.append((meta, toks[o:o + c].tolist(), lps[o:o + c].copy(), v0))
                self.n_tokens += c
                if not self.device_admit:
                    self.free.append(s_)
            self.done_seen += k
            if self.done_seen >= n_done:
                break
            self.harvest_begin()   # more records than one launch packs
        if self.device_admit:
            self._see_admissions(hdr)
            x = hdr[4 + 4 * self.hv_rows:]
            self.n_active_host = int(x[0])                                    # exact at the packing launch; only retirements since
            self.n_free_dev = self.B - int(x[0]) - (n_done - self.done_seen)  # finished rows not packed yet keep their slots
        else:
            self.n_active_host = self.n_active()
        return out

    def _see_admissions(self, hdr):
        """Device-side admission: the harvest header carries the number of prompts the device has admitted so far; the
        requests that crossed from staged to admitted since the last look get their start version."""
        if not self.device_admit:
            return
        head = int(hdr[4 + 4 * self.hv_rows + 1])
        while self.q_head < head:
            r = self.staged.popleft()
            self.meta[r] = (self.meta[r][0], self._admit_version)
            self.q_head += 1

    def poll(self):
        """Harvest now: harvest_begin() + harvest_end()."""
        if not self.harvest_pending:
            self.harvest_begin()
        return self.harvest_end()

    def chunk(self):
        """Fill idle slots from the queue, decode check_every steps, harvest (reference: StreamGen.chunk).  With
        overlap_harvest the harvest is only enqueued here and its results are returned by the next call, which takes them
        after it has enqueued its first decode step: the host's share of the harvest then costs no idle GPU time, and
        freed slots are refilled one step later."""
        steps, out = self.ce, []
        if self.harvest_pending:
            if self.n_active() > 0 and steps > 0:
                self.step()
                steps -= 1
            out = self.harvest_end()
        if self.device_admit:
            self._stage_prompts()
            while steps > 0 and self._admit_device():
                steps -= 1
        elif self.queue and self.free:
            if self.mixed and self.n_active() > 0:
                while self.queue and self.free and steps > 0 and self._admit_mixed():
                    steps -= 1
            else:
                self._admit()
        if self.n_active() == 0:
            return out
        for _ in range(steps):
            self.step()
        if self.overlap_harvest:
            self.harvest_begin()
            return out
        return out + self.poll()

    def run(self, max_chunks: int = 1 << 30):
        res = []
        for _ in range(max_chunks):
            if self.n_outstanding() == 0:
                break
            res += self.chunk()
        if self.harvest_pending:
            res += self.harvest_end()
        return res
