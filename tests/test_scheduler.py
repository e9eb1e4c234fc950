"""The scheduler's decisions (no GPU).  Scenarios after crates/prelude-core/src/scheduler/tests.rs."""
import random

import pytest

from prelude_amd.cache import PageTables
from prelude_amd.engine.scheduler import Scheduler, SchedulerError


def make(pages=1000, page=16, window_groups=(), **kw):
    tables = PageTables(page, [(pages, 0)] + [(pages, w) for w in window_groups])
    kw.setdefault("decode_priority_max_remaining_tokens", 0)
    return tables, Scheduler(tables, **kw)


def run_step(s, finish_after=None):
    """schedule, pretend the step ran, draw a token where one is due; returns the portions."""
    ps = s.schedule()
    s.step_done()
    for p in ps:
        if p.samples:
            s.on_token(p.id)
            info = s.info(p.id)
            if info.generated >= info.max_new or (finish_after and info.generated >= finish_after.get(p.id, 10 ** 9)):
                s.finish(p.id)
    return ps


def test_prefill_then_decode():
    # tests.rs:52-76
    _, s = make()
    s.add_request(1, 10, 3)
    ps = run_step(s)
    assert [(p.id, p.start, p.count, p.samples) for p in ps] == [(1, 0, 10, True)]
    ps = run_step(s)
    assert [(p.id, p.start, p.count, p.samples) for p in ps] == [(1, 10, 1, True)]
    ps = run_step(s)
    assert [(p.start, p.count) for p in ps] == [(11, 1)]       # third token; the request ends
    assert not s.has_work() and s.schedule() == []


def test_large_prefill_is_chunked_under_the_budget():
    # tests.rs:639-675: 250 tokens under a budget of 100 -> 100, 100, 50, then decode
    _, s = make(max_num_batched_tokens=100)
    s.add_request(1, 250, 5)
    got = [run_step(s)[0] for _ in range(4)]
    assert [(p.start, p.count, p.samples) for p in got] == [(0, 100, False), (100, 100, False), (200, 50, True), (250, 1, True)]


def test_decode_and_chunk_share_the_budget():
    # tests.rs:678-701: one decoding request costs 1, the newcomer gets 49 of 50
    _, s = make(max_num_batched_tokens=50)
    s.add_request(1, 10, 100)
    run_step(s)
    s.add_request(2, 200, 10)
    ps = run_step(s)
    assert [(p.id, p.count) for p in ps] == [(1, 1), (2, 49)]
    assert sum(p.count for p in ps) <= 50
    ps = run_step(s)
    assert [(p.id, p.start, p.count) for p in ps] == [(1, 11, 1), (2, 49, 49)]


def test_per_request_cap():
    # tests.rs:722-736
    _, s = make(max_num_batched_tokens=1000, long_prefill_token_threshold=64)
    s.add_request(1, 200, 2)
    s.add_request(2, 30, 2)
    ps = run_step(s)
    assert [(p.id, p.count) for p in ps] == [(1, 64), (2, 30)]


def test_a_request_of_its_own_portion_cap():
    # a cap that holds for one request only (its logits are wanted at every prompt position, say)
    _, s = make(max_num_batched_tokens=100)
    s.add_request(1, 70, 2, max_chunk=32)
    s.add_request(2, 70, 2)
    ps = run_step(s)
    assert [(p.id, p.start, p.count) for p in ps] == [(1, 0, 32), (2, 0, 68)]
    ps = run_step(s)
    assert [(p.id, p.start, p.count) for p in ps] == [(1, 32, 32), (2, 68, 2)]
    ps = run_step(s)
    assert [(p.id, p.start, p.count, p.samples) for p in ps] == [(1, 64, 6, True), (2, 70, 1, True)]


def test_a_request_fed_whole_or_not_at_all():
    """A request whose mixers cannot continue a prompt from a cut is never given a part of its prompt: it waits
    for a step that takes all of it, and after an eviction it is fed prompt and generated tokens whole again."""
    _, s = make(max_num_batched_tokens=64)
    s.add_request(1, 40, 30)
    run_step(s)                                   # 1 is decoding
    s.add_request(2, 62, 2, atomic=True)          # 62 + 1 decode token of request 1 = 63 <= 64: fits whole
    s.add_request(3, 30, 2, atomic=True)          # only 1 token of the budget is left: not cut, waits
    ps = run_step(s)
    assert [(p.id, p.start, p.count, p.samples) for p in ps] == [(1, 40, 1, True), (2, 0, 62, True)]
    ps = run_step(s)
    assert [(p.id, p.start, p.count) for p in ps] == [(1, 41, 1), (2, 62, 1), (3, 0, 30)]
    # what could never be fed whole is refused when it is added, with what a step takes
    with pytest.raises(SchedulerError, match="must be fed whole .70 tokens.*a step takes 64"):
        s.add_request(4, 60, 11, atomic=True)
    with pytest.raises(SchedulerError, match="a step takes 16"):
        s.add_request(5, 20, 1, atomic=True, max_chunk=16)
    # pages: a whole portion that the free pages cannot hold is not shortened
    tables, s = make(pages=6, page=16, max_num_batched_tokens=128, decode_reservation_cap=0)
    s.add_request(1, 60, 4)
    run_step(s)                                   # 4 pages held by request 1
    s.add_request(2, 50, 2, atomic=True)          # needs 4 pages, 2 are free: waits, whole
    ps = run_step(s)
    assert [(p.id, p.count) for p in ps] == [(1, 1)]
    for _ in range(2):
        assert [(p.id, p.count) for p in run_step(s)] == [(1, 1)]   # request 1 ends and gives its pages back
    ps = run_step(s)
    assert [(p.id, p.start, p.count, p.samples) for p in ps] == [(2, 0, 50, True)]
    assert tables.audit() == ""


def test_running_cap_and_fcfs():
    _, s = make(max_running_requests=2)
    for i in range(4):
        s.add_request(i, 5, 2)
    ps = run_step(s)
    assert [p.id for p in ps] == [0, 1] and s.num_waiting == 2
    ps = run_step(s)                                   # both finish (2 tokens each)
    assert [p.id for p in ps] == [0, 1]
    ps = run_step(s)
    assert [p.id for p in ps] == [2, 3]


def test_admission_is_by_pages_with_reserved_growth():
    # tests.rs:1089-1178: a newcomer is admitted only if its whole footprint fits beside what running prefills still owe
    t, s = make(pages=10, page=16, max_num_batched_tokens=32, decode_reservation_cap=16)
    s.add_request(1, 100, 4)       # needs ceil((100 + 4) / 16) = 7 pages in the end
    run_step(s)                    # first 32 tokens: 2 pages taken, 5 still owed
    assert t.live_pages(1, 0) == 2
    s.add_request(2, 40, 4)        # 3 pages; 8 free - 5 owed = 3 -> fits
    s.add_request(3, 20, 4)        # 2 pages more: does not fit beside them
    ps = run_step(s)
    assert [p.id for p in ps] == [1] and s.num_waiting == 2     # the budget went to request 1 first
    _, s2 = make(pages=10, page=16, max_num_batched_tokens=64, decode_reservation_cap=16)
    s2.add_request(1, 100, 4)
    run_step(s2)                   # 64 tokens: 4 pages, 3 owed
    s2.add_request(2, 40, 4)
    s2.add_request(3, 20, 4)
    ps = run_step(s2)              # 36 for request 1, then 28 of request 2; 3 (6 free - 0 owed... ) see below
    assert [p.id for p in ps][:2] == [1, 2]
    assert 3 not in [p.id for p in ps]


def test_request_that_can_never_fit_is_refused():
    _, s = make(pages=4, page=16)
    with pytest.raises(SchedulerError, match="pages"):
        s.add_request(1, 60, 10)
    s.add_request(2, 50, 14)       # exactly 64 tokens
    with pytest.raises(SchedulerError, match="already live"):
        s.add_request(2, 5, 1)
    with pytest.raises(SchedulerError, match="empty prompt"):
        s.add_request(3, 0, 1)


def test_pages_run_out_newest_is_evicted_and_recomputes_everything():
    # tests.rs:151, :1291-1350 -- decided here: the evicted request restarts with prompt and generated tokens
    t, s = make(pages=6, page=4, decode_reservation_cap=0)
    s.add_request(1, 8, 16)        # admitted on its prompt alone (reservation cap 0)
    s.add_request(2, 8, 16)
    run_step(s)                    # 2 + 2 pages
    assert s.num_running == 2
    evicted = False
    for _ in range(12):
        ps = run_step(s)
        assert ps, "the scheduler stalled"
        if s.last_preempted():
            assert s.last_preempted() == [2]           # never the oldest
            evicted = True
            info = s.info(2)
            assert info.computed == 0 and not info.running and info.preempt_count == 1 and info.generated > 0
            break
    assert evicted and t.audit() == ""
    # request 1 runs on; request 2 comes back later and feeds prompt + generated tokens from position 0
    seen_restart = False
    for _ in range(200):
        if not s.has_work():
            break
        ps = run_step(s)
        for p in ps:
            if p.id == 2 and p.start == 0:
                assert p.count > 8 or s.info(2).known > 8
                seen_restart = True
    assert seen_restart and not s.has_work() and t.free_pages(0) == 6


def test_short_decode_tail_holds_newcomers_back():
    # crates/prelude-core/src/scheduler/admission.rs:196-208
    _, s = make(decode_priority_max_remaining_tokens=4)
    s.add_request(1, 5, 3)
    run_step(s)                    # 2 tokens left
    s.add_request(2, 5, 3)
    ps = run_step(s)
    assert [p.id for p in ps] == [1]                   # within 4 tokens of its end: no admission
    ps = run_step(s)
    assert [p.id for p in ps] == [1]
    ps = run_step(s)
    assert [p.id for p in ps] == [2]


def test_window_groups_need_fewer_pages():
    t, s = make(pages=8, page=4, window_groups=(6,), max_num_batched_tokens=8)
    with pytest.raises(SchedulerError):
        s.add_request(1, 30, 10)                       # the full-attention group needs 10 pages
    t2 = PageTables(4, [(5, 6)])                       # only a windowed group
    s2 = Scheduler(t2, max_num_batched_tokens=4, decode_priority_max_remaining_tokens=0)
    s2.add_request(1, 40, 20)                          # 60 tokens through 5 pages of 4
    steps = 0
    while s2.has_work():
        assert run_step(s2)
        assert t2.audit() == ""
        steps += 1
    assert steps == 10 + 19 and t2.free_pages(0) == 5


@pytest.mark.parametrize("seed", range(5))
def test_every_request_finishes_and_nothing_leaks(seed):
    rng = random.Random(seed)
    page = rng.choice([4, 16])
    pages = rng.randint(12, 40)
    budget = rng.choice([8, 32, 100])
    t, s = make(pages=pages, page=page, max_num_batched_tokens=budget, max_running_requests=rng.choice([2, 4, 8]),
                long_prefill_token_threshold=rng.choice([0, 0, 16]), decode_reservation_cap=rng.choice([0, 8, 4096]),
                decode_priority_max_remaining_tokens=rng.choice([0, 4]))
    cap = pages * page
    want = {}
    nxt = 0
    fed = {}
    done = set()
    for _ in range(3000):
        if nxt < 25 and rng.random() < 0.3:
            plen = rng.randint(1, cap // 2)
            mx = rng.randint(1, max(1, cap - plen - 1))
            s.add_request(nxt, plen, mx)
            want[nxt] = (plen, mx)
            nxt += 1
        if not s.has_work():
            if nxt >= 25:
                break
            continue
        ps = s.schedule()
        assert ps, "stalled with work left"
        assert sum(p.count for p in ps) <= budget
        assert len({p.id for p in ps}) == len(ps)
        for rid in s.last_preempted():
            fed[rid] = 0
        for p in ps:
            assert p.start == fed.get(p.id, 0) and p.count >= 1
            fed[p.id] = p.start + p.count
            assert t.live_pages(p.id, 0) == -(-fed[p.id] // page)      # pages owned = ceil(kv_len / P)
        s.step_done()
        assert t.audit() == ""
        for p in ps:
            if p.samples:
                s.on_token(p.id)
                info = s.info(p.id)
                assert info.known == want[p.id][0] + info.generated
                if info.generated >= info.max_new or rng.random() < 0.02:
                    s.finish(p.id)
                    done.add(p.id)
    assert done == set(want) and not s.has_work()
    assert t.free_pages(0) == pages and t.num_requests() == 0
