"""Epoch model of the schedule of the streaming prefill kernel (flashck_amd/csrc/prefill_stream.hip): ring-buffer
safety, data landed before it is read, first-row cache hand-over, every tile read once.

`program()` restates the kernel's control flow (which requests, reads, waits and barriers a wave executes for a list of
items with given tile counts); `check()` then proves the invariants for that list.  It is a model of the algorithm, not
a run of the kernel: it guards the hand-off rules (when an item may prefetch the next one's tiles, how many requests a
wait may leave in flight, how many barriers a cold start needs) against changes made without a GPU at hand.

Each wave group runs the same program; op k of a group happens in epoch = number of barriers that group has passed.
Group 1 passes one extra barrier first, group 0 one extra at the end; barrier #j of both groups is the same event, so
an op of group a in epoch ea precedes an op of group b in epoch eb iff ea < eb (a != b); equal epochs = concurrent.
"""
import random

RING = 4


def program(ns):
    """ops of one group for items with tile counts ns; mirrors the control flow of prefill_stream_kernel"""
    ops = []
    pos = 0
    warm = False
    if ns:
        ops.append(("ROWW", 0))      # item 0's first rows, then the common barrier before the skew
        ops.append(("BAR",))
    for ii, n in enumerate(ns):
        has_next = ii + 1 < len(ns)
        nb = ns[ii + 1] if has_next else 0
        handoff = has_next and n >= 4 and nb >= 3
        if has_next:
            ops.append(("ROWW", ii + 1))

        def issue(opnd, want):
            if want < n or handoff:
                assert want < n or want - n < nb, "request past the next item"
                ops.append(("ROWR", ii if want < n else ii + 1))
                ops.append(("REQ", opnd, pos + want))

        if n > 0:
            if not warm:
                issue("K", 0); issue("V", 0); issue("K", 1); issue("K", 2); issue("V", 1)
                ops.append(("WAIT", 2 if (n >= 3 or handoff) else 0))
                ops.append(("BAR",)); ops.append(("BAR",))
                ops.append(("READ", "K", pos))          # M(-1): S = K0.Q
                ops.append(("BAR",))
            for i in range(n - 1):
                issue("K", i + 3); issue("V", i + 2)
                ops.append(("BAR",))                    # softmax(i); barrier
                ops.append(("READ", "V", pos + i)); ops.append(("READ", "K", pos + i + 1))
                ops.append(("WAIT", 2 if (handoff or i + 3 < n) else 0))
                ops.append(("BAR",))
            if handoff:
                issue("K", n + 2); issue("V", n + 1)
            ops.append(("BAR",))                        # softmax(n-1); barrier
            ops.append(("READ", "V", pos + n - 1))
            if handoff:
                ops.append(("READ", "K", pos + n))
                ops.append(("WAIT", 2))
            else:
                ops.append(("WAIT", 0))
            ops.append(("BAR",))
        else:
            ops.append(("BAR",)); ops.append(("BAR",))  # an item without tiles still separates the row-cache write from its readers
        pos += n
        warm = handoff
    return ops


def check(ns):
    prog = program(ns)
    # per group: epoch of every op, landing epoch of every request
    per = []
    for g in (0, 1):
        epoch = 0
        ev = []
        queue = []  # outstanding requests (index into ev)
        skewed = False
        for op in prog:
            if op[0] == "BAR":
                epoch += 1
                if g == 1 and not skewed:
                    epoch += 1   # the skew: group 1 passes one more barrier right after the first common one
                    skewed = True
                continue
            if op[0] == "REQ":
                ev.append(dict(kind="REQ", opnd=op[1], p=op[2], e=epoch, land=None))
                queue.append(len(ev) - 1)
            elif op[0] in ("ROWW", "ROWR"):
                ev.append(dict(kind=op[0], item=op[1], e=epoch))
            elif op[0] == "WAIT":
                while len(queue) > op[1]:
                    ev[queue.pop(0)]["land"] = epoch
            else:
                ev.append(dict(kind="READ", opnd=op[1], p=op[2], e=epoch, order=len(ev)))
        assert not queue, f"requests still in flight at the end: {[ev[q] for q in queue]}"
        per.append(ev)
    nbar = sum(1 for op in prog if op[0] == "BAR")
    # both groups pass nbar + 1 barriers in total (group 1: one extra first, group 0: one extra last)
    # group 1 ops: the extra barrier first means its op epochs are shifted by +1 relative to barrier numbering
    # (handled by the initial epoch above: group 0 op after j barriers is in global epoch j, group 1's in j + 1)
    for g in (0, 1):
        for k, x in enumerate(per[g]):
            if x["kind"] in ("ROWW", "ROWR"):
                continue
            if x["kind"] == "READ":
                # 1. every request of that tile has landed before the read
                for gg in (0, 1):
                    reqs = [r for r in per[gg] if r["kind"] == "REQ" and r["opnd"] == x["opnd"] and r["p"] == x["p"]]
                    assert len(reqs) == 1, f"tile {x['opnd']}{x['p']} requested {len(reqs)} times by group {gg} (ns={ns})"
                    r = reqs[0]
                    if gg == g:
                        assert r["land"] <= x["e"] and per[g].index(r) < k, f"own share not landed: {r} before {x} ns={ns}"
                        # the wait precedes the read in program order: waits sit before the barrier that precedes the read
                        assert r["land"] < x["e"], f"own wait not before the barrier: {r} {x} ns={ns}"
                    else:
                        assert r["land"] < x["e"], f"other group's share may not have landed: {r} vs read {x} ns={ns}"
            else:
                # 2. the buffer a request overwrites is no longer read by anyone
                for gg in (0, 1):
                    for y in per[gg]:
                        if y["kind"] == "READ" and y["opnd"] == x["opnd"] and y["p"] < x["p"] and (x["p"] - y["p"]) % RING == 0:
                            if gg == g:
                                assert y["e"] <= x["e"] and per[g].index(y) < k, f"own read after overwrite: {y} {x} ns={ns}"
                            else:
                                assert y["e"] < x["e"], f"overwrite races with the other group's read: req {x} (group {g}) vs read {y} (group {gg}) ns={ns}"
    # 2b. first-row cache: two halves, item i in half i % 2; LDS writes by all threads, so every order needs a barrier
    for g in (0, 1):
        for x in per[g]:
            if x["kind"] == "ROWR":
                for gg in (0, 1):
                    w = [y for y in per[gg] if y["kind"] == "ROWW" and y["item"] == x["item"]]
                    assert len(w) == 1 and w[0]["e"] < x["e"], f"first rows of item {x['item']} read before written: {w} {x} ns={ns}"
            if x["kind"] == "ROWW":
                for gg in (0, 1):
                    for y in per[gg]:
                        if y["kind"] == "ROWR" and y["item"] < x["item"] and (x["item"] - y["item"]) % 2 == 0:
                            assert y["e"] < x["e"], f"first rows of item {y['item']} overwritten while read: {y} {x} ns={ns}"
    # 3. every tile of every item is read exactly once per operand and group
    want = []
    p = 0
    for n in ns:
        want += [("K", p + t) for t in range(n)] + [("V", p + t) for t in range(n)]
        p += n
    for g in (0, 1):
        got = sorted((x["opnd"], x["p"]) for x in per[g] if x["kind"] == "READ")
        assert got == sorted(want), f"reads differ ns={ns}"
    return nbar


def test_fixed_item_lists():
    for ns in ([1], [2], [3], [4], [5], [4, 3], [4, 4], [8, 3, 4, 9], [4, 2], [3, 8], [0, 5], [5, 0, 5], [1, 1, 1],
               [12, 12, 12], [0], [0, 0, 4], [40, 40]):
        check(ns)


def test_random_item_lists():
    rng = random.Random(1)
    for _ in range(400):
        check([rng.choice([0, 1, 2, 3, 4, 5, 6, 7, 9, 17, 40]) for _ in range(rng.randint(1, 7))])


def test_the_model_rejects_broken_schedules():
    """The checks have teeth: a ring of three buffers, a single barrier after a cold start's wait, or a wait that leaves
    two batches in flight are all caught."""
    import pytest
    global RING
    RING = 3
    try:
        with pytest.raises(AssertionError, match="overwrite races"):
            check([12, 12, 12])
    finally:
        RING = 4
    src = open(__file__).read().split("def test_fixed_item_lists")[0]
    for old, new, what in (
            ('ops.append(("BAR",)); ops.append(("BAR",))\n                ops.append(("READ", "K", pos))', 'ops.append(("BAR",))\n                ops.append(("READ", "K", pos))', "may not have landed"),
            ('ops.append(("WAIT", 2 if (handoff or i + 3 < n) else 0))', 'ops.append(("WAIT", 4 if (handoff or i + 3 < n) else 0))', "not before the barrier|not landed"),
            ("handoff = has_next and n >= 4 and nb >= 3", "handoff = has_next and n >= 4 and nb >= 1", "past the next item")):
        assert old in src, old
        ns = {}
        exec(compile(src.replace(old, new), "mutant", "exec"), ns)
        with pytest.raises(AssertionError, match=what):
            for case in ([4, 4], [8, 3, 4, 9], [12, 12, 12], [5], [3, 8], [6, 1, 7], [9, 2]):
                ns["check"](case)


def _deal(total, nwx):
    """Work-list dealing of the kernel: rank k of the valid slots goes to workgroup snake(k) at list position 2*round (+1)."""
    lists = {w: {} for w in range(nwx)}
    for k in range(total):
        m = k % (2 * nwx)
        for wgx in range(nwx):
            which = 0 if m == wgx else (1 if m == 2 * nwx - 1 - wgx else -1)
            if which >= 0:
                lists[wgx][2 * (k // (2 * nwx)) + which] = k
    counts = {}
    for wgx in range(nwx):
        rem = total % (2 * nwx)
        counts[wgx] = 2 * (total // (2 * nwx)) + (1 if rem > wgx else 0) + (1 if rem > 2 * nwx - 1 - wgx else 0)
    return lists, counts


def test_work_list_dealing_is_a_partition_with_dense_ordered_lists():
    for nwx in (1, 2, 3, 32):
        for total in list(range(0, 4 * nwx + 3)) + [824, 1000]:
            lists, counts = _deal(total, nwx)
            seen = sorted(k for l in lists.values() for k in l.values())
            assert seen == list(range(total)), (nwx, total)                    # every valid slot, exactly once
            for wgx, l in lists.items():
                assert sorted(l) == list(range(counts[wgx])), (nwx, total, wgx)  # positions 0..count-1, no holes
                ranks = [l[p] for p in sorted(l)]
                assert ranks == sorted(ranks)                                    # heaviest (lowest rank) first
            assert max(counts.values()) - min(counts.values()) <= 2
            assert max(counts.values()) <= total // nwx + 2                     # bound the launcher sizes the list with


def test_work_list_balance_on_descending_costs():
    # costs sorted in descending order (row tiles, heaviest first), as the slot order provides them
    rng = random.Random(3)
    for _ in range(20):
        costs = sorted((rng.randint(1, 128) for _ in range(rng.randint(200, 2000))), reverse=True)
        nwx = 32
        lists, _ = _deal(len(costs), nwx)
        loads = [sum(costs[k] for k in l.values()) for l in lists.values()]
        assert max(loads) <= 1.05 * (sum(costs) / nwx) + 128
