"""Pins oracle.sched: brute force against a straight-line per-request loop and the reference's rollout invariants
(tests/test_rl_stream.py:82-94: every request returned exactly once, rows EOS-terminated or exactly the limit long)."""
import numpy as np

from oracle.sched import SlotTable


def _stream(req, n, V=50, eos=1):
    """Deterministic fake model: token t of request r."""
    rng = np.random.default_rng(1000 + req)
    return rng.integers(0, V, size=n)


def test_slot_table_matches_per_request_loop():
    B, max_new, eos, n_req = 8, 24, 1, 40
    rng = np.random.default_rng(0)
    limits = rng.integers(1, max_new + 1, size=n_req)
    expect = {}
    for r in range(n_req):
        s = _stream(r, max_new)
        row = list(s[:limits[r]])
        if eos in row:
            row = row[:row.index(eos) + 1]
        expect[r] = row
    tab = SlotTable(B, max_new, eos)
    free, nxt, got, seen = list(range(B))[::-1], 0, {}, 0
    for step in range(400):
        while free and nxt < n_req:                     # admit FIFO into free slots
            s = free.pop()
            tab.admit([s], [nxt], [limits[nxt]], [_stream(nxt, max_new)[0]], [0.0], [5], [0])
            nxt += 1
        for r, s, c in tab.done[seen:]:                 # harvest
            got[r] = tab.out_tok[s, :c].tolist()
            free.append(s)
        seen = len(tab.done)
        if nxt == n_req and not (tab.req >= 0).any():
            break
        slot, d, n_act = tab.compact(B)
        assert n_act == (tab.req >= 0).sum() and list(slot[:n_act]) == sorted(slot[:n_act])
        new = [_stream(d["req"][i], max_new)[d["cnt"][i]] if slot[i] >= 0 else 0 for i in range(B)]
        pos_before = tab.pos.copy()
        tab.commit(slot, new, np.zeros(B, np.float32))
        for i in range(n_act):
            s = slot[i]
            assert tab.pos[s] in (0, pos_before[s] + 1)   # advanced, or parked on retirement
    assert sorted(got) == list(range(n_req))
    assert got == expect
    for r, row in got.items():
        assert row[-1] == eos or len(row) == limits[r]
    assert (tab.pos == 0).all() and (tab.req == -1).all()


def test_bucket_smaller_than_active_and_retire_probability():
    tab = SlotTable(6, 16)
    tab.admit(list(range(6)), list(range(6)), [16] * 6, [3] * 6, [0.0] * 6, [4] * 6, [0] * 6)
    slot, d, n_act = tab.compact(4)
    assert n_act == 6 and list(slot) == [0, 1, 2, 3]
    tab2 = SlotTable(512, 64)
    tab2.admit(list(range(512)), list(range(512)), [64] * 512, [3] * 512, [0.0] * 512, [4] * 512, [0] * 512)
    slot, d, _ = tab2.compact(512)
    tab2.commit(slot, [5] * 512, np.zeros(512, np.float32), retire_p=0.25, seed=7)
    frac = len(tab2.done) / 512
    assert 0.17 < frac < 0.33


def test_expand_prompts_matches_vectorised_construction():
    """The loop restatement against an independent vectorised construction (np.repeat of per-prompt values, the way the
    reference's prefill_packed_host forms its index tensors, fast_decode.py:219-236) on random ragged prompt sets."""
    import numpy as np
    from oracle.sched import expand_prompts
    rng = np.random.default_rng(0)
    for _ in range(50):
        A = int(rng.integers(1, 9))
        lens = rng.integers(1, 30, size=A)
        cu = np.concatenate([[0], np.cumsum(lens)])
        slots = rng.permutation(20)[:A]
        starts = rng.integers(0, 10, size=A)
        n_tok = int(cu[-1]) + int(rng.integers(0, 8))
        pos, row, last, last_idx, bind = expand_prompts(cu, slots, starts, n_tok)
        seg = np.repeat(np.arange(A), lens)
        N = int(cu[-1])
        assert np.array_equal(pos[:N], np.arange(N) - cu[:-1][seg] + starts[seg])
        assert np.array_equal(row[:N], slots[seg]) and np.array_equal(last[:N], (starts + lens - 1)[seg])
        assert (row[N:] == -1).all() and (pos[N:] == 0).all()
        assert np.array_equal(last_idx, cu[1:] - 1)
        assert bind == {int(s): (int(a), int(a + n)) for s, a, n in zip(slots, starts, lens)}


def test_plan_admit_policy_properties():
    """What defines the device-side admission without restating it: the admitted prompts are a prefix of the queue; they get
    the lowest-numbered reusable slots (not active, not held) in ascending order; the prefix is maximal - it stops only when
    the queue, the reusable slots, the prompt cap or the token budget is exhausted; the packed tokens are the prompts back to
    back; with left padding all admitted prompts end at the same position."""
    rng = np.random.default_rng(3)
    for trial in range(200):
        B, A, Np = int(rng.integers(1, 40)), int(rng.integers(1, 9)), int(rng.integers(4, 80))
        tab = SlotTable(B, 8)
        tab.req[:] = np.where(rng.random(B) < 0.5, rng.integers(0, 1000, size=B), -1)
        tab.hold[:] = (tab.req < 0) & (rng.random(B) < 0.3)
        queue = [(rng.integers(1, 99, size=int(rng.integers(1, 24))).tolist(), 5000 + i, int(rng.integers(1, 9))) for i in range(int(rng.integers(0, 12)))]
        head = int(rng.integers(0, len(queue) + 1))
        left = bool(trial % 2)
        cu, slot, start, limit, req, tok, new_head = tab.plan_admit(queue, head, A, Np, left)
        na = new_head - head
        assert 0 <= na <= A and list(req[:na]) == [q[1] for q in queue[head:new_head]] and list(limit[:na]) == [q[2] for q in queue[head:new_head]]
        reusable = [s for s in range(B) if tab.req[s] < 0 and not tab.hold[s]]
        assert list(slot[:na]) == reusable[:na] and (slot[na:] == -1).all()
        lens = [len(q[0]) for q in queue[head:new_head]]
        assert list(np.diff(cu[:na + 1])) == lens and (cu[na:] == sum(lens)).all() and sum(lens) <= Np
        assert list(tok[:sum(lens)]) == [t for q in queue[head:new_head] for t in q[0]] and (tok[sum(lens):] == 0).all()
        # maximal: one more prompt would break a limit
        assert na == A or new_head == len(queue) or na == len(reusable) or sum(lens) + len(queue[new_head][0]) > Np
        if left and na:
            assert len({int(start[a]) + lens[a] for a in range(na)}) == 1 and min(start[:na]) == 0
        else:
            assert (start == 0).all()


def test_device_admission_loop_returns_every_request_once():
    """The slot table driven only through plan_admit / commit / harvest (no host free list): every request exactly once, rows
    as the per-request loop expects, and a slot is never handed out while its finished row waits for the harvest."""
    B, max_new, eos, n_req, A, Np = 6, 16, 1, 30, 3, 40
    rng = np.random.default_rng(5)
    limits = rng.integers(1, max_new + 1, size=n_req)
    prompts = [rng.integers(2, 50, size=int(rng.integers(1, 20))).tolist() for _ in range(n_req)]
    expect = {}
    for r in range(n_req):
        row = list(_stream(r, max_new)[:limits[r]])
        expect[r] = row[:row.index(eos) + 1] if eos in row else row
    tab = SlotTable(B, max_new, eos)
    queue = [(prompts[r], r, int(limits[r])) for r in range(n_req)]
    head, got = 0, {}
    for step in range(600):
        if step % 3 == 0:                                   # harvest cadence: slower than retirement
            for r, s, c, tk, lp in tab.harvest(2):
                assert r not in got
                got[r] = tk.tolist()
        waiting = {s for _, s, _ in tab.done[tab.harvested:]}
        cu, slot, start, limit, req, tok, head = tab.plan_admit(queue, head, A, Np, False)
        na = int((slot >= 0).sum())
        assert not (set(slot[:na].tolist()) & waiting)      # held slots are never reused
        if na:
            tab.admit(slot[:na], req[:na], limit[:na], [_stream(int(r), max_new)[0] for r in req[:na]], [0.0] * na,
                      [cu[a + 1] - cu[a] for a in range(na)], start[:na])
        if head == n_req and not (tab.req >= 0).any() and tab.harvested == len(tab.done):
            break
        sl, d, n_act = tab.compact(B)
        new = [_stream(d["req"][i], max_new)[d["cnt"][i]] if sl[i] >= 0 else 0 for i in range(B)]
        tab.commit(sl, new, np.zeros(B, np.float32))
    assert got == expect
