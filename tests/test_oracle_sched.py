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
