"""The cache manager (no page lost, held twice or freed twice, under random
orders of requests; windows give pages back) and the scheduler's decisions
(decode first, portions under the token budget, preemption when pages run
out).  No GPU."""
import random

import pytest

from tiny_llm_infer_amd.cache import CacheFull, CacheManager, CacheNeed, PageError, PagePool
from tiny_llm_infer_amd.engine.scheduler import Scheduler, SchedulerConfig, SchedulerError
from tiny_llm_infer_amd.engine.sequence import Sequence, Status
from tiny_llm_infer_amd.sampling.params import SamplingParams

FULL = CacheNeed.keys_and_values(2, 16, None)
WIN = CacheNeed.keys_and_values(2, 16, 20)


# --------------------------------------------------------------------- pages --
def test_pool_hands_out_the_lowest_free_page_and_refuses_double_release():
    pool = PagePool(4)
    assert [pool.take() for _ in range(3)] == [0, 1, 2]
    pool.release(1)
    assert pool.take() == 1
    pool.release(0)
    with pytest.raises(PageError):
        pool.release(0)
    with pytest.raises(PageError):
        pool.release(9)
    assert pool.take() == 0 and pool.take() == 3
    with pytest.raises(PageError):
        pool.take()
    pool.check()


def test_reviving_a_page_never_queues_it_twice():
    """A page taken back by id and released again, many times over: the queue of free ids
    holds every id at most once (it does not grow), the lowest free id still comes first."""
    pool = PagePool(6)
    assert [pool.take() for _ in range(6)] == list(range(6))
    for p in (4, 2, 5):
        pool.release(p)
    for _ in range(50):
        pool.revive(2)
        pool.check()
        pool.release(2)
        pool.revive(5)
        pool.release(5)
    pool.check()
    assert len(pool._heap) <= 6
    assert [pool.take() for _ in range(3)] == [2, 4, 5]
    with pytest.raises(PageError):
        pool.take()
    pool.check()


def test_a_cache_need_names_its_records():
    from tiny_llm_infer_amd.cache import PAGE, CacheRecord
    kv = CacheNeed.keys_and_values(2, 16, None)
    assert [(r.name, r.page_shape(8)) for r in kv.records] == [("k", (2, 8, 16)), ("v", (2, 16, 8))]
    assert kv == FULL and kv != WIN and sum(r.elems_per_token() for r in kv.records) == 64
    with pytest.raises(ValueError):
        CacheRecord("x", (4, 4))                # no axis for the page's tokens
    with pytest.raises(ValueError):
        CacheNeed((CacheRecord("x", (PAGE, 4)), CacheRecord("x", (PAGE, 2))))
    # layers whose records differ do not share a group
    m = CacheManager([FULL, CacheNeed((CacheRecord("latent", (PAGE, 24)),), None), FULL], 8, 4, 1)
    assert [g.cache_layers for g in m.groups] == [[0, 2], [1]]


def test_groups_have_pages_of_their_own():
    m = CacheManager([FULL, WIN, FULL, None, WIN], page_size=8, num_pages=10, max_requests=2)
    assert [g.cache_layers for g in m.groups] == [[0, 2], [1, 4]]
    m.admit("a")
    m.reserve("a", 20)
    assert m.free_pages() == [7, 7]
    assert m.get("a").tables[0] == [0, 1, 2] and m.get("a").tables[1] == [0, 1, 2]
    m.release("a")
    assert m.free_pages() == [10, 10]
    m.check()


def test_window_pages_are_given_back_when_passed():
    m = CacheManager([FULL, WIN], page_size=8, num_pages=64, max_requests=1)
    m.admit("a")
    m.reserve("a", 50)
    m.advance("a", 50)
    # the next query is at 50 and reads 31..50: blocks 0..2 (slots 0..23) are passed
    assert list(m.get("a").tables[1][:4]) == [-1, -1, -1, 3]
    assert list(m.get("a").tables[0][:4]) == [0, 1, 2, 3]
    held = 64 - m.free_pages()[1]
    assert held == 4
    for n in range(51, 200):
        m.reserve("a", n)
        m.advance("a", n)
        live = [p for p in m.get("a").tables[1] if p >= 0]
        assert len(live) <= 20 // 8 + 2          # the window, not the history
        first = (n - 20 + 1) // 8
        assert all(p < 0 for p in m.get("a").tables[1][:first])
        assert all(p >= 0 for p in m.get("a").tables[1][first:(n + 7) // 8])
    m.check()
    m.release("a")
    assert m.free_pages() == [64, 64]


def test_reserve_is_all_or_nothing():
    m = CacheManager([FULL, WIN], page_size=8, num_pages=3, max_requests=2)
    m.admit("a")
    m.admit("b")
    m.reserve("a", 16)
    assert not m.can_reserve("b", 17)
    with pytest.raises(CacheFull):
        m.reserve("b", 17)
    assert m.free_pages() == [1, 1] and m.get("b").tables == [[], []]
    m.reserve("b", 8)
    with pytest.raises(ValueError):
        m.advance("b", 9)                         # more than was reserved
    with pytest.raises(CacheFull):
        m.admit("c")                              # no slot
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_no_page(seed):
    rng = random.Random(seed)
    m = CacheManager([FULL, WIN, FULL, WIN], page_size=4, num_pages=40, max_requests=5)
    live = {}
    taken_slots = set()
    for it in range(600):
        r = rng.random()
        if r < 0.2 and len(live) < 5:
            key = f"q{it}"
            rc = m.admit(key)
            assert rc.slot not in taken_slots
            taken_slots.add(rc.slot)
            live[key] = 0
        elif r < 0.85 and live:
            key = rng.choice(list(live))
            n = live[key] + rng.choice([1, 1, 1, 2, 5, 9, 17])
            if m.can_reserve(key, n):
                m.reserve(key, n)
                m.advance(key, n)
                live[key] = n
            else:
                with pytest.raises(CacheFull):
                    m.reserve(key, n)
        elif live:
            key = rng.choice(list(live))
            taken_slots.discard(m.get(key).slot)
            m.release(key)
            del live[key]
        m.check()
        # every token a later query may read is held
        for key, n in live.items():
            rc = m.get(key)
            for gi, g in enumerate(m.groups):
                lo = 0 if g.need.window is None else max(0, n - g.need.window + 1)
                for pos in range(lo, n):
                    assert rc.tables[gi][pos // 4] >= 0
    for key in list(live):
        m.release(key)
    m.check()
    assert m.free_pages() == [40, 40]
    assert m.pages_taken_total == m.pages_returned_total > 80      # pages were used again


def test_a_window_group_gets_no_more_pages_than_its_requests_can_hold():
    """Given the most tokens a step brings, a window group's pool is the smaller one: for every
    live request the window's blocks and two for the edges, and a step's tokens on top."""
    from tiny_llm_infer_amd.cache.manager import group_needs, window_group_pages
    assert window_group_pages(20, 8, 3, 64) == 3 * (3 + 2) + 8
    m = CacheManager([FULL, WIN, FULL], page_size=8, num_pages=500, max_requests=3, max_step_tokens=64)
    assert m.pages_per_group() == [500, 23] and m.num_pages == 500
    assert CacheManager([FULL, WIN], 8, 10, 3, max_step_tokens=64).pages_per_group() == [10, 10]    # never more than asked
    assert CacheManager([FULL, WIN], 8, 500, 3).pages_per_group() == [500, 500]                    # nothing known about steps
    assert CacheManager([WIN, FULL], 8, [7, 9], 1).pages_per_group() == [7, 9]                     # one count a group
    assert group_needs([WIN, None, FULL, WIN]) == [WIN, FULL]
    with pytest.raises(ValueError, match="page counts"):
        CacheManager([WIN, FULL], 8, [7], 1)
    # what one request holds at most: everything where all keys are kept, window + portion where not
    assert m.most_pages_needed(1000, 64) == [125, 3 + 2 + 8]
    assert m.most_pages_needed(30, 64) == [4, 4]


@pytest.mark.parametrize("seed", range(4))
def test_the_smaller_window_pool_is_never_the_one_that_runs_out(seed):
    """Random requests run in random portions, three live at a time, a step's portions within
    its token budget: the window group's pool, sized as above, always has the pages."""
    rng = random.Random(seed)
    budget, live_max = 48, 3
    m = CacheManager([FULL, WIN], page_size=4, num_pages=4000, max_requests=live_max, max_step_tokens=budget)
    assert m.pages_per_group()[1] == live_max * (5 + 2) + 12
    live, low = {}, m.pages_per_group()[1]
    for it in range(400):
        while len(live) < live_max:
            key = f"q{it}-{len(live)}-{rng.random()}"
            m.admit(key)
            live[key] = [0, rng.randrange(1, 300)]
        left = budget
        for key in list(live):
            at, size = live[key]
            n = min(size - at, left, rng.choice([1, 1, 2, 5, 17, 48]))
            if n <= 0:
                continue
            left -= n
            m.reserve(key, at + n)                     # (raises CacheFull if the window pool were too small)
            low = min(low, m.free_pages()[1])
            live[key][0] = at + n
        for key in list(live):
            m.advance(key, live[key][0])
            if live[key][0] == live[key][1]:
                m.release(key)
                del live[key]
        m.check()
    assert low < 12                                    # the pool was nearly used up, so the bound is no loose one


# ----------------------------------------------------------------- scheduler --
def _seq(i, n, max_tokens=4):
    return Sequence(i, list(range(n)), n, SamplingParams(max_tokens=max_tokens, ignore_eos=True))


def _run(sched, plan, token=1):
    """Pretend the model ran: advance the cache and post-process."""
    for item in plan.items:
        s = item.seq
        sched.cache.reserve(s.request_id, item.first + item.count)
        sched.cache.advance(s.request_id, item.first + item.count)
    return sched.postprocess(plan, [token if i.samples else None for i in plan.items], lambda t: False)


def test_prompts_are_cut_to_the_token_budget_one_portion_a_step():
    cache = CacheManager([FULL], page_size=8, num_pages=100, max_requests=4)
    s = Scheduler(SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=24), cache)
    a, b = _seq(1, 50), _seq(2, 10)
    s.add(a)
    s.add(b)
    p = s.schedule()
    assert [(i.seq.request_id, i.first, i.count, i.prompt_portion) for i in p.items] == \
        [(1, 0, 24, True)]
    _run(s, p)
    p = s.schedule()          # b is now first in the queue, a went to the back
    assert [(i.seq.request_id, i.first, i.count) for i in p.items] == \
        [(2, 0, 10), (1, 24, 14)]
    assert [i.samples for i in p.items] == [True, False]
    _run(s, p)
    assert b.status == Status.RUNNING and b.size == 11
    p = s.schedule()          # decode first, then the rest of a's prompt
    assert [(i.seq.request_id, i.first, i.count, i.prompt_portion) for i in p.items] == \
        [(2, 10, 1, False), (1, 38, 12, True)]
    assert p.num_tokens == 13
    _run(s, p)
    p = s.schedule()
    assert [(i.seq.request_id, i.prompt_portion) for i in p.items] == [(2, False), (1, False)]


def test_max_num_seqs_limits_a_step_and_running_requests_take_turns():
    cache = CacheManager([FULL], page_size=8, num_pages=100, max_requests=8)
    s = Scheduler(SchedulerConfig(max_num_seqs=2, max_num_batched_tokens=100), cache)
    for i in range(1, 4):
        s.add(_seq(i, 5, max_tokens=10))
    p = s.schedule()
    assert [i.seq.request_id for i in p.items] == [1, 2]
    _run(s, p)
    p = s.schedule()          # two running requests fill the step; 3 waits
    assert [i.seq.request_id for i in p.items] == [1, 2]
    _run(s, p)


def test_requests_finish_at_max_tokens_or_eos_and_give_everything_back():
    cache = CacheManager([FULL, WIN], page_size=8, num_pages=10, max_requests=2)
    s = Scheduler(SchedulerConfig(2, 64), cache)
    a = Sequence(1, [5, 6, 7], 3, SamplingParams(max_tokens=3))
    b = Sequence(2, [5, 6], 2, SamplingParams(max_tokens=50))
    s.add(a)
    s.add(b)
    done = []
    for step in range(3):
        p = s.schedule()
        for item in p.items:
            cache.reserve(item.seq.request_id, item.first + item.count)
            cache.advance(item.seq.request_id, item.first + item.count)
        # b draws the end-of-sequence token 99 in the second step
        toks = [99 if (i.seq is b and step == 1) else 1 for i in p.items]
        done += s.postprocess(p, toks, lambda t: t == 99)
    assert [d.request_id for d in done] == [2, 1]
    assert b.completion_tokens == [1, 99] and a.completion_tokens == [1, 1, 1]
    assert s.is_finished() and cache.free_pages() == [10, 10] and cache.free_slots() == 2
    cache.check()


def test_when_pages_run_out_the_request_is_preempted_and_computed_again():
    cache = CacheManager([FULL], page_size=4, num_pages=4, max_requests=4)
    s = Scheduler(SchedulerConfig(4, 64), cache)
    a, b = _seq(1, 7, max_tokens=8), _seq(2, 7, max_tokens=8)
    s.add(a)
    s.add(b)
    _run(s, s.schedule())                       # both prompts: 2 pages each, pool full
    assert cache.free_pages() == [0]
    p = s.schedule()                            # both decode at position 7: still fits
    assert len(p.items) == 2
    _run(s, p)
    p = s.schedule()                            # position 8 needs a third page: a is preempted,
    assert s.num_preemptions == 1               # its pages let b go on
    assert [(i.seq.request_id, i.prompt_portion) for i in p.items] == [(2, False)]
    assert a.status == Status.WAITING and not a.admitted and a.preemptions == 1
    assert s.waiting[0] is a
    _run(s, p)
    # b runs to its end; then a is admitted again and recomputes prompt + generated tokens
    while b.status != Status.FINISHED:
        _run(s, s.schedule())
    p = s.schedule()
    assert [(i.seq.request_id, i.first, i.count, i.prompt_portion) for i in p.items] == \
        [(1, 0, 9, True)]
    while not s.is_finished():
        _run(s, s.schedule())
    assert a.completion_size == 8 and b.completion_size == 8
    assert cache.free_pages() == [4]
    cache.check()


def test_a_prompt_larger_than_the_pool_is_an_error_and_a_stuck_queue_too():
    cache = CacheManager([FULL], page_size=4, num_pages=2, max_requests=2)
    s = Scheduler(SchedulerConfig(2, 64), cache)
    s.add(_seq(1, 9))
    with pytest.raises(SchedulerError, match="more than all"):
        s.schedule()
    cache = CacheManager([FULL], page_size=4, num_pages=2, max_requests=2)
    cache.admit("someone else")
    cache.reserve("someone else", 8)
    s = Scheduler(SchedulerConfig(2, 64), cache)
    s.add(_seq(1, 5))
    with pytest.raises(SchedulerError, match="nothing can run"):
        s.schedule()


def _launch(sched, plan):
    """What putting a step on the device does to the cache (the host's side of it)."""
    for item in plan.items:
        sched.cache.reserve(item.seq.request_id, item.first + item.count)
        sched.cache.advance(item.seq.request_id, item.first + item.count)


def _shape(plan):
    return [(i.seq.request_id, i.first, i.count, i.prompt_portion) for i in plan.items]


def test_a_step_planned_ahead_goes_on_with_prompts_beside_decoding():
    """While a step runs, the next one is planned from what that step will leave: the request
    whose prompt ends in it decodes (its token is still on the device), the other's prompt goes
    on after the portion that runs.  A request that is not admitted yet ends the look ahead."""
    cache = CacheManager([FULL], page_size=8, num_pages=100, max_requests=4)
    s = Scheduler(SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=24), cache)
    a, b = _seq(1, 50), _seq(2, 10)
    s.add(a)
    s.add(b)
    p0 = s.schedule()
    assert _shape(p0) == [(1, 0, 24, True)]
    _launch(s, p0)
    assert s.plan_ahead(p0) is None           # b is next and holds nothing yet
    s.postprocess(p0, [None], lambda t: False)
    p1 = s.schedule()                         # b first (a went to the back), then a from token 24 on
    assert _shape(p1) == [(2, 0, 10, True), (1, 24, 14, True)]
    _launch(s, p1)
    p2 = s.plan_ahead(p1)                     # b decodes at position 10 with the token p1 samples
    assert _shape(p2) == [(2, 10, 1, False), (1, 38, 12, True)]
    assert [i.samples for i in p2.items] == [True, True] and p2.num_tokens == 13
    assert a.status == Status.RUNNING and list(s.running) == [b, a] and not s.waiting
    assert a.tokens_in_cache == 24            # what p1 and p2 run is counted when their results come in
    _launch(s, p2)
    s.postprocess(p1, [7, None], lambda t: False)
    assert b.token_ids[-1] == 7 and b.size == 11 and a.tokens_in_cache == 38
    p3 = s.plan_ahead(p2)                     # both decode, fed on the device
    assert _shape(p3) == [(2, 11, 1, False), (1, 50, 1, False)]
    _launch(s, p3)
    s.postprocess(p2, [8, 9], lambda t: False)
    c = _seq(3, 5)
    s.add(c)                                  # arrives now: not admitted, so the next plan waits for p3's end
    assert s.plan_ahead(p3) is None
    s.postprocess(p3, [8, 9], lambda t: False)
    assert _shape(s.schedule()) == [(2, 12, 1, False), (1, 51, 1, False), (3, 0, 5, True)]
    cache.check()


@pytest.mark.parametrize("seed", range(12))
def test_steps_planned_ahead_are_the_steps_planned_afterwards(seed):
    """Two schedulers serve the same random requests (several groups of layers, small pools,
    budgets from 2 tokens, arrivals on the way): one plans every step after the one before has
    been post-processed, the other plans ahead wherever ``plan_ahead`` gives a plan.  Without
    end-of-sequence tokens both run the same steps, and no page is lost."""
    rng = random.Random(300 + seed)
    needs = [FULL, WIN] if rng.random() < 0.5 else [FULL]
    page = rng.choice([4, 8, 16])
    budget = rng.choice([2, 5, 16, 40])
    nreq = rng.randrange(1, 9)
    lens = [rng.randrange(1, 90) for _ in range(nreq)]
    outs = [rng.randrange(1, 9) for _ in range(nreq)]
    most = max((n + o + page - 1) // page for n, o in zip(lens, outs)) + 1
    pages = rng.choice([most, most + 2, 3 * most, most * nreq + 2])
    seqs = rng.randrange(1, 6)
    arrive = [rng.randrange(0, 12) for _ in range(nreq)]

    def serve(ahead):
        cache = CacheManager(needs, page_size=page, num_pages=pages, max_requests=seqs, max_step_tokens=budget)
        s = Scheduler(SchedulerConfig(max_num_seqs=seqs, max_num_batched_tokens=budget), cache)

        def arrivals(n):                      # the requests that are there when plan number n is made
            for i in range(nreq):
                if arrive[i] == n:
                    s.add(_seq(i, lens[i], max_tokens=outs[i]))

        plans, planned_ahead, inflight = [], 0, None
        for n in range(2000):
            if inflight is None:
                arrivals(n)
                if s.is_finished():
                    if n > max(arrive):
                        break
                    plans.append([])
                    continue
                inflight = s.schedule()
                _launch(s, inflight)
            cur, inflight = inflight, None
            plans.append(_shape(cur))
            if ahead:
                before = len(s.waiting)
                arrivals(n + 1)
                inflight = s.plan_ahead(cur)
                if inflight is not None:
                    planned_ahead += 1
                    _launch(s, inflight)
                else:                         # they arrive again when the plan is made the ordinary way
                    while len(s.waiting) > before:
                        s.waiting.pop()
            s.postprocess(cur, [1 if i.samples else None for i in cur.items], lambda t: False)
            cache.check()
        assert s.is_finished() and cache.free_pages() == cache.pages_per_group()
        return plans, planned_ahead

    plain, _ = serve(False)
    looked, planned_ahead = serve(True)
    assert looked == plain


# ------------------------------------------------------------ prefix caching --
def test_page_hash_is_chained_fnv1a():
    from tiny_llm_infer_amd.cache.manager import page_hash
    # FNV-1a, 64 bit, over 8 bytes of the previous hash then 4 bytes per token, little-endian
    h = 1469598103934665603
    for byte in [0] * 8 + [7, 0, 0, 0, 1, 1, 0, 0]:
        h = ((h ^ byte) * 1099511628211) % (1 << 64)
    assert page_hash([7, 257], 0) == h
    assert page_hash([7, 257], 1) != h and page_hash([257, 7], 0) != h


def test_prefix_pages_are_shared_revived_and_forgotten():
    m = CacheManager([FULL, FULL], page_size=4, num_pages=8, max_requests=3, prefix_caching=True)
    a = list(range(100, 111))                     # 11 tokens: 2 full pages + 3
    m.admit("a")
    assert m.adopt_prefix("a", a) == 0
    m.reserve("a", 11)
    m.advance("a", 11)
    m.register_pages("a", a)
    # b shares a's first two pages while a is live; its third page is its own
    b = a[:8] + [1, 2, 3]
    m.admit("b")
    assert m.adopt_prefix("b", b) == 8
    assert m.get("b").tables[0] == list(m.get("a").tables[0][:2])
    assert m.groups[0].pool.ref_count(m.get("a").tables[0][0]) == 2
    m.reserve("b", 11)
    assert m.get("b").tables[0][2] != m.get("a").tables[0][2]
    m.advance("b", 11)
    m.check()
    # never the last page: a prompt of exactly 8 tokens still computes its second page
    m.admit("c")
    assert m.adopt_prefix("c", a[:8]) == 4
    m.release("c")
    m.release("a")
    m.release("b")
    assert m.free_pages() == [8]
    # free pages are revived by id ...
    m.admit("d")
    assert m.adopt_prefix("d", a) == 8 and m.prefix_hits == 2 + 1 + 2
    m.release("d")
    # ... until the pool hands them out for something else
    m.admit("e")
    m.reserve("e", 32)
    m.release("e")
    m.admit("f")
    assert m.adopt_prefix("f", a) == 0
    m.release("f")
    m.check()
    with pytest.raises(ValueError):
        CacheManager([FULL, WIN], page_size=4, num_pages=8, max_requests=1, prefix_caching=True)


def test_a_block_table_reads_like_a_list_and_is_one_piece_of_memory():
    """What the step function relies on when it packs the tables of a step: the table can be
    viewed as int32 memory without a conversion, and goes on growing afterwards."""
    import numpy as np
    from tiny_llm_infer_amd.cache.manager import PageTable
    t = PageTable()
    assert len(t) == 0 and not t and t == []
    for page in (7, 3, 9):
        t.append(page)
    assert t == [7, 3, 9] and t != [7, 3] and list(t[:2]) == [7, 3] and t[1] == 3
    assert list(reversed(t)) == [9, 3, 7]
    row = np.full(8, -1, dtype=np.int32)
    row[:len(t)] = np.frombuffer(t, dtype=np.int32)
    assert row.tolist() == [7, 3, 9, -1, -1, -1, -1, -1]
    t[0] = -1                      # a window has passed the page
    t.append(11)                   # no view is held any more: the table grows
    assert t == [-1, 3, 9, 11]


def test_layers_with_a_window_take_their_pages_portion_by_portion():
    """An admitted request holds all the pages of its prompt where all keys are kept, and in a
    window group only what the next portion needs: a long prompt passes through a window pool
    that could never hold it whole."""
    cache = CacheManager([FULL, WIN], page_size=8, num_pages=200, max_requests=2, max_step_tokens=32)
    assert cache.pages_per_group() == [200, 2 * 5 + 4]
    s = Scheduler(SchedulerConfig(max_num_seqs=2, max_num_batched_tokens=32), cache)
    a, b = _seq(1, 400, max_tokens=3), _seq(2, 90, max_tokens=3)
    s.add(a)
    s.add(b)
    steps = 0
    while not s.is_finished():
        p = s.schedule()
        assert p.items and p.num_tokens <= 32
        held = [n - f for n, f in zip(cache.pages_per_group(), cache.free_pages())]
        assert held[1] <= 14
        _run(s, p)
        cache.check()
        steps += 1
    assert a.completion_size == 3 and b.completion_size == 3 and s.num_preemptions == 0
    assert cache.free_pages() == [200, 14]
    # a request too long for the pool of the layers that keep all keys is still an error
    s.add(_seq(3, 8 * 200 + 1))
    with pytest.raises(SchedulerError, match="more than all"):
        s.schedule()
