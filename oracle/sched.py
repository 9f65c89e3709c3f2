"""Continuous-batching slot bookkeeping, pure-Python simulator (checker only; see oracle/__init__.py).

Restates the slot logic of the reference's host loops (generate_continuous, ultraviolet/model.py:1283-1350; StreamGen,
scripts/rl_stream.py:66-146) at per-step granularity, which is what the device-side table does: the token drawn from
the prefill is token 0 of a request (model.py:1306-1313); a row finishes when its count reaches its limit or it emits
EOS, inclusive (rl_stream.py:131-138); finished rows are parked at position 0 (model.py:1345-1350); the output column is
clamped to the buffer width (rl_stream.py:122).  The reference tests a row only every check_every steps and discards
what it decoded past the end; retiring at the exact step returns the same rows.

Device-side admission (plan_admit / harvest with holds) restates the refill policy of the same loops - idle rows are
refilled from the head of a FIFO queue (rl_stream.py:76-93; model.py:1293-1314) - with two choices the reference leaves to
Python list order made explicit: free slots are handed out in ascending order, and a slot whose finished row has not been
harvested yet is not handed out.

Pinned by: the invariants of the reference's tests (every request returned once, rows EOS-terminated or exactly limit
long: tests/test_rl_stream.py:82-94) and brute-force comparison with a straight-line per-request loop in
tests/test_oracle_sched.py.
"""
from __future__ import annotations

import numpy as np

from . import philox


class SlotTable:
    def __init__(self, B: int, max_new: int, eos_id: int | None = None):
        self.B, self.max_new, self.eos = B, max_new, -1 if eos_id is None else int(eos_id)
        self.req = np.full(B, -1, np.int64)
        self.cnt = np.zeros(B, np.int64)
        self.limit = np.zeros(B, np.int64)
        self.tok = np.zeros(B, np.int64)
        self.pos = np.zeros(B, np.int64)
        self.starts = np.zeros(B, np.int64)
        self.out_tok = np.zeros((B, max_new), np.int32)
        self.out_lp = np.zeros((B, max_new), np.float32)
        self.done: list[tuple[int, int, int]] = []   # (request, slot, count)
        self.hold = np.zeros(B, np.int32)            # finished, output row not harvested yet: not reusable
        self.harvested = 0                           # completion records already packed

    def _finish(self, slot, req, cnt):
        self.done.append((int(req), int(slot), int(cnt)))
        self.req[slot] = -1
        self.hold[slot] = 1
        self.pos[slot] = 0
        self.starts[slot] = 0

    def admit(self, slots, req_ids, limits, first_tok, first_lp, pos, starts):
        for i, s in enumerate(slots):
            self.req[s], self.limit[s], self.tok[s], self.cnt[s] = req_ids[i], limits[i], first_tok[i], 1
            self.pos[s], self.starts[s] = pos[i], starts[i]
            self.out_tok[s, 0], self.out_lp[s, 0] = first_tok[i], first_lp[i]
            if limits[i] <= 1 or (self.eos >= 0 and first_tok[i] == self.eos):
                self._finish(s, req_ids[i], 1)

    def compact(self, n_bucket: int):
        act = np.nonzero(self.req >= 0)[0]
        n = min(len(act), n_bucket)
        out = {k: np.zeros(n_bucket, np.int64) for k in ("tok", "pos", "starts", "req", "cnt")}
        slot = np.full(n_bucket, -1, np.int64)
        slot[:n] = act[:n]
        for k, src in (("tok", self.tok), ("pos", self.pos), ("starts", self.starts), ("req", self.req), ("cnt", self.cnt)):
            out[k][:n] = src[act[:n]]
        return slot, out, len(act)

    def commit(self, act_slot, new_tok, new_lp, retire_p: float = 0.0, seed: int = 0):
        for i, s in enumerate(act_slot):
            if s < 0:
                continue
            c = int(self.cnt[s])
            col = min(c, self.max_new - 1)
            self.out_tok[s, col], self.out_lp[s, col] = new_tok[i], new_lp[i]
            self.cnt[s], self.tok[s] = c + 1, new_tok[i]
            self.pos[s] += 1
            fin = c + 1 >= self.limit[s] or (self.eos >= 0 and new_tok[i] == self.eos)
            if not fin and retire_p > 0:
                fin = float(philox.request_uniform(seed, int(self.req[s]), c, philox.DOMAIN_RETIRE)) < np.float32(retire_p)
            if fin:
                self._finish(s, self.req[s], c + 1)


    def harvest(self, max_rows: int):
        """Pack the next completion records (at most max_rows) and release their slots: [(request, slot, count, tokens,
        log-probs)]."""
        out = []
        for req, slot, cnt in self.done[self.harvested:self.harvested + max_rows]:
            c = min(cnt, self.max_new)
            out.append((req, slot, c, self.out_tok[slot, :c].copy(), self.out_lp[slot, :c].copy()))
            self.hold[slot] = 0
        self.harvested += len(out)
        return out

    def plan_admit(self, queue, head: int, admit_cap: int, n_tokens: int, left_pad: bool):
        """The admission of one step: queue[head:] are the staged prompts in arrival order, each (tokens, request id, limit).
        Prompts are taken from the head while a reusable slot is left (not active, not held), at most admit_cap prompts and
        n_tokens packed tokens; the k-th admitted prompt gets the k-th free slot in ascending order.  Returns the tables of
        the step: cu_seqlens (admit_cap + 1, unused entries repeat the total), slot (-1 unused), start, limit, request id
        per prompt, the packed tokens (zero filled), and the new head."""
        free = [s for s in range(self.B) if self.req[s] < 0 and not self.hold[s]][:admit_cap]
        na, ntok, lens = 0, 0, []
        while na < len(free) and head + na < len(queue):
            n = len(queue[head + na][0])
            if ntok + n > n_tokens:
                break
            ntok += n
            lens.append(n)
            na += 1
        tmax = max(lens, default=0)
        cu = np.full(admit_cap + 1, ntok, np.int64)
        cu[:na + 1] = np.concatenate([[0], np.cumsum(lens)]) if na else [0]
        slot = np.full(admit_cap, -1, np.int64)
        start, limit, req = (np.zeros(admit_cap, np.int64) for _ in range(3))
        tok = np.zeros(n_tokens, np.int64)
        for a in range(na):
            ids, r, lim = queue[head + a]
            slot[a], limit[a], req[a] = free[a], lim, r
            start[a] = tmax - lens[a] if left_pad else 0
            tok[cu[a]:cu[a + 1]] = ids
        return cu, slot, start, limit, req, tok, head + na


def expand_prompts(cu, slots, starts, n_tokens: int):
    """Per-token tables of a packed prefill, as the reference builds them on the host (prefill_packed_host,
    ultraviolet/kernels/fast_decode.py:210-269): for packed token i of prompt a (cu[a] <= i < cu[a+1]) its position
    starts[a] + i - cu[a], its cache row slots[a] and the last position of its prompt starts[a] + len[a] - 1; tokens at or
    after cu[-1] are padding (row -1, position 0).  Also the packed index of every prompt's last token (0 for an empty or
    unused entry, slot < 0) and the (start, end) positions of every admitted slot.  Plain loops."""
    cu = [int(c) for c in cu]
    A = len(cu) - 1
    pos = np.zeros(n_tokens, np.int64)
    row = np.full(n_tokens, -1, np.int64)
    last = np.zeros(n_tokens, np.int64)
    last_idx = np.zeros(A, np.int64)
    bind = {}
    for a in range(A):
        n = cu[a + 1] - cu[a]
        if n <= 0 or slots[a] < 0:
            continue
        for i in range(cu[a], min(cu[a + 1], n_tokens)):
            pos[i] = starts[a] + i - cu[a]
            row[i] = slots[a]
            last[i] = starts[a] + n - 1
        last_idx[a] = cu[a + 1] - 1
        bind[int(slots[a])] = (int(starts[a]), int(starts[a] + n))
    return pos, row, last, last_idx, bind
