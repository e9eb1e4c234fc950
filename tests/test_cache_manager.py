"""The cache manager's bookkeeping (no GPU): no page lost, held twice or freed twice, under random orders of requests."""
import random

import numpy as np
import pytest

from prelude_amd.cache import CacheError, OutOfPages, PageTables


def test_allocate_free_and_exhaustion():
    # scenarios of crates/prelude-core/src/scheduler/components/cache/block_manager.rs:112-199
    t = PageTables(16, [(4, 0)])
    t.open(1)
    t.reserve(1, 33)                       # 33 tokens -> 3 pages
    assert t.free_pages(0) == 1 and len(t.table(1, 0)) == 3
    t.commit(1, 33)
    t.open(2)
    with pytest.raises(OutOfPages):
        t.reserve(2, 17)                   # needs 2, 1 free: nothing is taken
    assert t.free_pages(0) == 1 and t.table(2, 0) == [] and t.audit() == ""
    t.reserve(2, 16)
    assert t.free_pages(0) == 0
    t.close(1)
    assert t.free_pages(0) == 3 and t.audit() == ""
    with pytest.raises(CacheError):
        t.close(1)                         # never freed twice silently
    t.close(2)
    assert t.free_pages(0) == 4 and t.num_requests() == 0


def test_slot_formula():
    # crates/prelude-core/src/scheduler/components/cache/block_manager.rs:151-158
    table = [5, 10, 3]
    assert [PageTables.slot(table, p, 16) for p in (0, 15, 16, 33)] == [80, 95, 160, 49]


def test_pages_are_reused_first_in_first_out():
    t = PageTables(8, [(3, 0)])
    t.open(1); t.reserve(1, 24); t.commit(1, 24)
    assert t.table(1, 0) == [0, 1, 2]
    t.close(1)
    t.open(2); t.reserve(2, 9); t.commit(2, 9)
    assert t.table(2, 0) == [0, 1]
    t.open(3); t.reserve(3, 1)
    assert t.table(3, 0) == [2]


def test_misuse_is_refused():
    t = PageTables(8, [(8, 0)])
    t.open(1)
    with pytest.raises(CacheError, match="already live"):
        t.open(1)
    t.reserve(1, 5)
    with pytest.raises(CacheError, match="in flight"):
        t.reserve(1, 9)
    with pytest.raises(CacheError):
        t.commit(1, 4)
    t.commit(1, 5)
    with pytest.raises(CacheError, match="cannot extend"):
        t.reserve(1, 5)
    with pytest.raises(CacheError, match="not live"):
        t.reserve(7, 5)
    t.reserve(1, 20)
    t.rollback(1)                          # the step did not run
    assert t.length(1) == 5 and len(t.table(1, 0)) == 1 and t.free_pages(0) == 7 and t.audit() == ""


def test_window_gives_pages_back_early():
    t = PageTables(4, [(100, 0), (100, 6)])     # group 1 looks back over 6 keys
    t.open(1)
    pos = 0
    for n in (5, 2, 9, 1, 1, 1, 7, 1):
        t.reserve(1, pos + n)
        # every key a query of this portion can see still has its page
        table = t.table(1, 1)
        first_key = max(0, pos - 6 + 1)
        for key in range(first_key, pos + n):
            assert table[key // 4] >= 0
        # pages wholly before the first visible key are gone
        for i, p in enumerate(table):
            if (i + 1) * 4 <= first_key:
                assert p == -1
        assert all(p >= 0 for p in t.table(1, 0))
        pos += n
        t.commit(1, pos)
        assert t.audit() == ""
    assert t.live_pages(1, 0) == 7 and t.live_pages(1, 1) <= 3
    assert t.free_pages(1) == 100 - t.live_pages(1, 1)
    t.close(1)
    assert t.free_pages(0) == 100 and t.free_pages(1) == 100


def test_all_groups_or_none():
    t = PageTables(4, [(10, 0), (2, 0)])
    t.open(1)
    with pytest.raises(OutOfPages):
        t.reserve(1, 12)                   # group 1 has 2 pages, 3 needed
    assert t.free_pages(0) == 10 and t.free_pages(1) == 2


def test_state_slots():
    t = PageTables(4, [(10, 0)], state_slots=2)
    t.open(1, need_state=True)
    t.open(2, need_state=True)
    assert {t.state_slot(1), t.state_slot(2)} == {0, 1} and t.free_state_slots() == 0
    with pytest.raises(CacheError, match="state slot"):
        t.open(3, need_state=True)
    t.open(4)                              # a request without state needs none
    assert t.state_slot(4) == -1
    t.close(1)
    t.open(3, need_state=True)
    assert t.free_state_slots() == 0 and t.audit() == ""


def _fill(t, ids, starts, counts):
    n, total = len(ids), sum(counts)
    stride = max(-(-(s + c) // t.page_size) for s, c in zip(starts, counts))
    layout = t.step_layout(n, total, stride, 0)
    buf = np.full(layout["_total"][1], -7, dtype=np.int32)
    t.fill_step(ids, starts, counts, stride, buf, layout)
    get = lambda k: buf[layout[k][0]: layout[k][0] + layout[k][1]]
    return get, stride


def test_step_arrays():
    t = PageTables(4, [(16, 0), (16, 5)], state_slots=4)
    t.open(10, True); t.reserve(10, 6); t.commit(10, 6)
    t.open(11, True); t.reserve(11, 3)
    t.reserve(10, 7)
    get, stride = _fill(t, [11, 10], [0, 6], [3, 1])
    assert stride == 2
    assert get("positions").tolist() == [0, 1, 2, 6] and get("seq_of_token").tolist() == [0, 0, 0, 1]
    assert get("cu_q").tolist() == [0, 3, 4] and get("context_lens").tolist() == [3, 7]
    assert get("fresh").tolist() == [1, 0]
    assert get("state_slots").tolist() == [t.state_slot(11), t.state_slot(10)]
    bt = get("block_tables").reshape(2, 2, 2)
    assert bt[0, 0].tolist() == t.table(11, 0) + [-1] and bt[0, 1].tolist() == t.table(10, 0)
    slots = get("slots").reshape(2, 4)
    for g in range(2):
        assert slots[g].tolist() == [PageTables.slot(t.table(11, g), p, 4) for p in range(3)] + \
            [PageTables.slot(t.table(10, g), 6, 4)]
    # position <-> (page, offset) is a bijection within a table
    t.commit(11, 3); t.commit(10, 7)
    t.reserve(10, 40)
    get, _ = _fill(t, [10], [7], [33])
    s0 = get("slots").reshape(2, 33)[0].tolist()
    assert len(set(s0)) == 33
    with pytest.raises(CacheError, match="does not continue"):
        _fill(t, [10], [8], [32])


def runs_of(table):
    """Lengths of the stretches of a table whose pages lie side by side in the pool."""
    out, n = [], 0
    for i, p in enumerate(table):
        if i and p == table[i - 1] + 1:
            n += 1
        else:
            if n:
                out.append(n)
            n = 1
    return out + ([n] if n else [])


def test_requests_that_grow_in_turn_get_their_pages_in_runs():
    """Pages of 16 tokens are handed out in runs of 8 (128 tokens) where whole runs are free: four requests that
    grow a page at a time, in turn, each end up with their pages side by side, not interleaved."""
    t = PageTables(16, [(64, 0)])
    for r in range(4):
        t.open(r)
    for n in range(1, 16):
        for r in range(4):
            t.reserve(r, 16 * n); t.commit(r, 16 * n)
        assert t.audit() == ""
    for r in range(4):
        table = t.table(r, 0)
        assert len(table) == 15 and runs_of(table) == [8, 7], table
    assert t.free_pages(0) == 4                      # what the four keep in reserve is free all the same
    # a fifth request finds no whole run: it is given the pages that have been free the longest, one by one,
    # though each of them is kept for someone else -- and then the pool is empty, as it would be without runs
    t.open(9); t.reserve(9, 64); t.commit(9, 64)
    assert t.free_pages(0) == 0 and t.audit() == ""
    with pytest.raises(OutOfPages):
        t.reserve(0, 16 * 16)
    t.close(9)
    t.reserve(0, 16 * 16); t.commit(0, 16 * 16)      # the page behind its last one is free again: a run of 8 + 8
    assert runs_of(t.table(0, 0)) == [8, 8]
    for r in range(4):
        t.close(r)
    assert t.free_pages(0) == 64 and t.audit() == ""
    # everything is free and unclaimed again: a new request gets whole runs from the start
    t.open(5); t.reserve(5, 16 * 20); t.commit(5, 16 * 20)
    assert max(runs_of(t.table(5, 0))) >= 8 and t.audit() == ""


def test_a_request_that_ends_gives_up_what_was_kept_for_it():
    t = PageTables(16, [(16, 0)])
    t.open(1); t.reserve(1, 16); t.commit(1, 16)     # takes page 0, pages 1..7 are kept for it
    t.open(2); t.reserve(2, 16); t.commit(2, 16)     # takes page 8, pages 9..15 are kept for it
    assert t.table(1, 0) == [0] and t.table(2, 0) == [8]
    t.close(1)                                       # run 0 is whole again
    t.open(3); t.reserve(3, 48); t.commit(3, 48)
    assert t.table(3, 0) == [0, 1, 2] and t.audit() == ""
    t.reserve(2, 32); t.commit(2, 32)
    assert t.table(2, 0) == [8, 9]


@pytest.mark.parametrize("seed", range(10))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    page = rng.choice([1, 4, 8, 16])
    big = seed >= 6                                  # pools of several runs of 128 tokens
    groups = [(rng.randint(6, 40) * (6 if big else 1), 0), (rng.randint(6, 40) * (6 if big else 1), rng.choice([3, 9, 20]))]
    t = PageTables(page, groups, state_slots=3)
    live = {}
    nxt = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            need = rng.random() < 0.5 and t.free_state_slots() > 0
            t.open(nxt, need)
            live[nxt] = 0
            nxt += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 13, 30] + ([70, 200] if big else []))
            before = [t.free_pages(g) for g in range(2)]
            try:
                t.reserve(rid, live[rid] + n)
            except OutOfPages:
                # nothing taken beyond what the window released
                assert all(t.free_pages(g) >= before[g] for g in range(2))
                assert t.reservable_len(rid) < live[rid] + n
            else:
                if rng.random() < 0.15:
                    t.rollback(rid)
                else:
                    live[rid] += n
                    t.commit(rid, live[rid])
                    assert t.length(rid) == live[rid]
        elif live:
            rid = rng.choice(list(live))
            t.close(rid)
            del live[rid]
        assert t.audit() == "", t.audit()
        for g in range(2):
            held = sum(t.live_pages(r, g) for r in live)
            assert held + t.free_pages(g) == groups[g][0]
            for r in live:   # full-attention group: exactly ceil(len / page) pages
                if g == 0 and t.length(r) == live[r]:
                    assert t.live_pages(r, 0) == -(-live[r] // page)
    for rid in list(live):
        t.close(rid)
    assert [t.free_pages(g) for g in range(2)] == [g[0] for g in groups] and t.free_state_slots() == 3


def test_a_long_session_does_not_pile_up_stale_queue_entries():
    """Requests that always find the page behind their last one (a lightly used pool) never make the pool fall
    back to its first-in first-out queue, which is the only place stale entries used to be dropped: the audit
    fails when a queue holds more than about twice what it can validly hold, and it must stay fast."""
    import time
    t = PageTables(16, [(1024, 0)])
    for i in range(20000):
        t.open(i)
        t.reserve(i, 128)                  # eight pages: a whole run
        t.commit(i, 128)
        t.close(i)
        if i % 5000 == 4999:
            assert t.audit() == ""
    t0 = time.time()
    assert t.audit() == "" and t.free_pages(0) == 1024
    assert time.time() - t0 < 0.5
    # with a window pages come back one at a time while the request lives
    t = PageTables(4, [(64, 8)])
    t.open(0)
    for n in range(1, 6000):
        t.reserve(0, n)
        t.commit(0, n)
    assert t.audit() == ""


def test_pool_sizes_per_group():
    """A group with a window needs pages for what a window and a portion span, per request that may run; the
    Python rule used to size the pools is the manager's own."""
    from prelude_amd.cache.manager import pages_per_group, peak_pages
    from prelude_amd.parts.base import KVCacheSpec
    t = PageTables(8, [(100, 0), (100, 24), (100, 5)])
    for total in (1, 7, 8, 9, 63, 64, 500):
        for chunk in (1, 2, 8, 13, 64, 1000):
            for g, w in enumerate((0, 24, 5)):
                assert peak_pages(total, chunk, w, 8) == t.peak_pages(total, chunk, g), (total, chunk, w)
    groups = [KVCacheSpec(2, 16, 0), KVCacheSpec(2, 16, 24), KVCacheSpec(1, 32, 5)]
    # 4,096 tokens for at most 4 requests fed 16 tokens at a time: 512 pages where every key is kept,
    # 4 * (ceil((16 + 23) / 8) + 1) = 24 and 4 * (ceil((16 + 4) / 8) + 1) = 16 where a window passes
    assert pages_per_group(4096, groups, 8, max_requests=4, max_request_tokens=2048, chunk=16) == [512, 24, 16]
    # never more than the tokens asked for, never less than a page
    assert pages_per_group(40, groups, 8, max_requests=4, max_request_tokens=2048, chunk=16) == [5, 5, 5]
    assert pages_per_group(1, groups, 8, max_requests=1, max_request_tokens=8, chunk=1) == [1, 1, 1]


def test_a_value_width_of_its_own_counts_in_the_bytes():
    """A mixer whose values are narrower (or wider) than its keys: a group of its own, and the bytes a token takes
    follow both widths."""
    import torch
    from prelude_amd.cache.manager import bytes_per_token, plan_groups
    from prelude_amd.parts import KVCacheSpec
    same, narrow = KVCacheSpec(2, 64, 0), KVCacheSpec(2, 64, 0, value_dim=16)
    assert same.v_dim == 64 and narrow.v_dim == 16
    groups, of_slot = plan_groups([same, narrow, same])
    assert groups == [same, narrow] and of_slot == [0, 1, 0]
    assert bytes_per_token([same, narrow], torch.bfloat16) == 2 * (64 + 64) * 2 + 2 * (64 + 16) * 2
