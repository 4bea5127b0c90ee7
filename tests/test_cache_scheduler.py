"""The cache manager's bookkeeping and the scheduler's decisions (no GPU).
The scheduler is driven with a stand-in for the model that "samples" a fixed
function of the request and position, so its plans can be checked exactly."""

import random
import zlib

import pytest

from fastgen_amd.cache import RELEASED, CacheManager, OutOfPages, OutOfSlots
from fastgen_amd.engine.scheduler import Request, Scheduler


# ------------------------------------------------------------ cache manager
def test_pages_follow_the_length():
    c = CacheManager(16, [8], [None], n_slots=2)
    c.admit("a")
    c.reserve("a", 17)
    assert c.block_table("a") == [0, 1] and c.free_pages() == 6
    c.advance("a", 17)
    c.reserve("a", 15)  # fills page 1 exactly
    assert len(c.block_table("a")) == 2
    c.advance("a", 15)
    c.reserve("a", 1)
    assert len(c.block_table("a")) == 3
    assert c.write_slots("a", 0, 30, 3).tolist() == [1 * 16 + 14, 1 * 16 + 15, 2 * 16 + 0]
    c.check()
    with pytest.raises(RuntimeError, match="without reserved pages"):
        c.advance("a", 40)


def test_freed_pages_are_used_again_last_freed_first():
    c = CacheManager(16, [4], [None], n_slots=3)
    for r in "ab":
        c.admit(r)
        c.reserve(r, 32)
        c.advance(r, 32)
    assert c.free_pages() == 0
    c.admit("c")
    with pytest.raises(OutOfPages, match="needs 1 more pages in cache group 0, 0 are free"):
        c.reserve("c", 1)
    assert c.block_table("c") == []  # all or nothing
    pages_a = c.block_table("a")
    c.release("a")
    c.reserve("c", 20)
    assert sorted(c.block_table("c")) == sorted(pages_a)
    assert c.block_table("c")[0] == pages_a[-1]  # the page freed last is on top
    c.check()
    with pytest.raises(KeyError):
        c.release("a")  # freed twice


def test_slots():
    c = CacheManager(16, [4], [None], n_slots=2)
    s = {c.admit("a"), c.admit("b")}
    assert s == {0, 1}
    with pytest.raises(OutOfSlots):
        c.admit("c")
    with pytest.raises(KeyError, match="already live"):
        c.admit("a")
    c.release("a")
    assert c.admit("c") in s
    c.check()


def test_window_group_gives_pages_back():
    # group 0 keeps all keys, group 1 a window of 20 tokens
    c = CacheManager(8, [32, 32], [None, 20], n_slots=1)
    c.admit("a")
    n = 0
    for step in [5, 30, 1, 1, 17, 2, 64, 1]:
        c.reserve("a", step)
        # during the step the first new token at position n still reads keys n-19 .. n
        lo = max(0, n - 20 + 1) // 8
        assert all(p != RELEASED for p in c.block_table("a", 1)[lo:])
        c.advance("a", step)
        n += step
        c.check()
        tbl = c.block_table("a", 1)
        first_needed = max(0, n - 20 + 1) // 8
        assert all(p == RELEASED for p in tbl[:first_needed]) and all(p != RELEASED for p in tbl[first_needed:])
        assert RELEASED not in c.block_table("a", 0)
    assert c.free_pages(1) == 32 - sum(p != RELEASED for p in c.block_table("a", 1))
    assert c.free_pages(1) > c.free_pages(0)
    c.release("a")
    assert c.free_pages(0) == c.free_pages(1) == 32


@pytest.mark.parametrize("seed", range(6))
def test_no_page_lost_held_twice_or_freed_twice_under_random_orders(seed):
    rng = random.Random(seed)
    c = CacheManager(16, [24, 24], [None, 40], n_slots=5)
    live, n_next = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            rid = f"r{n_next}"
            n_next += 1
            c.admit(rid)
            live[rid] = 0
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 7, 16, 33])
            if c.can_reserve(rid, n):
                c.reserve(rid, n)
                c.advance(rid, n)
                live[rid] += n
                assert c.length(rid) == live[rid]
            else:
                with pytest.raises(OutOfPages):
                    c.reserve(rid, n)
        elif live:
            rid = rng.choice(list(live))
            c.release(rid)
            del live[rid]
        c.check()
        held = {p for r in live for p in c.block_table(r, 0)}
        assert len(held) + c.free_pages(0) == 24
    for rid in list(live):
        c.release(rid)
    c.check()
    assert c.free_pages(0) == c.free_pages(1) == 24 and c.free_slots() == 5


# ---------------------------------------------------------------- scheduler
def fake_token(req, pos):
    """The stand-in model's token at ``pos`` of a request: 3..98, the same in every process (``hash`` of a string
    is not), so that ids 0..2 and 99 never come by chance."""
    return zlib.crc32(f"{req.rid}:{pos}".encode()) % 96 + 3


def drive(sched, max_steps=10_000):
    """Run the scheduler to the end with the stand-in model; returns the plans."""
    plans = []
    for _ in range(max_steps):
        if not sched.has_work():
            break
        plan = sched.plan()
        sched.finished.clear()
        if not plan:
            continue
        assert sum(e.n for e in plan) <= sched.max_step_tokens
        assert len({e.request.rid for e in plan}) == len(plan)
        for e in plan:
            assert e.start == e.request.n_fed == sched.cache.length(e.request.rid)
            assert e.wants_logits == (e.start + e.n == e.request.n_known())
            sched.cache.advance(e.request.rid, e.n)
        sched.cache.check()
        plans.append([(e.request.rid, e.start, e.n, e.wants_logits) for e in plan])
        sched.commit(plan, [fake_token(e.request, e.start + e.n) for e in plan if e.wants_logits])
    else:
        raise AssertionError("the scheduler did not finish")
    return plans


def mk(cache_pages=64, page=16, max_batch=4, budget=24, max_seq=None, admit_reserve=0):
    c = CacheManager(page, [cache_pages], [None], n_slots=max_batch)
    return Scheduler(c, max_batch, budget, max_seq, admit_reserve=admit_reserve)


def test_budget_decodes_first_then_prompt_portions():
    s = mk(budget=24)
    reqs = [Request(i, list(range(n)), max_new=4) for i, n in enumerate([5, 17, 33])]
    for r in reqs:
        s.add(r)
    plans = drive(s)
    # step 0: 5 + 17 + the first 2 of request 2 = 24 tokens
    assert plans[0] == [(0, 0, 5, True), (1, 0, 17, True), (2, 0, 2, False)]
    # step 1: requests 0 and 1 decode one token each, request 2 gets the other 22
    assert plans[1] == [(0, 5, 1, True), (1, 17, 1, True), (2, 2, 22, False)]
    assert plans[2] == [(0, 6, 1, True), (1, 18, 1, True), (2, 24, 9, True)]
    for r in reqs:
        assert len(r.generated) == 4 and r.finish_reason == "length"
        assert r.generated == [fake_token(r, len(r.prompt) + i) for i in range(4)]
    assert s.cache.live_requests() == [] and s.cache.free_pages() == 64


def test_cut_on_a_prompt_end_and_prompt_of_one():
    """A budget that ends exactly on a prompt's end (fastgen/generate.py:815-817
    holds one token back there; here the portion simply ends the prompt and
    asks for its logits) and a prompt of one token."""
    s = mk(budget=8)
    a, b = Request("a", list(range(8)), 2), Request("b", [7], 3)
    s.add(a), s.add(b)
    plans = drive(s)
    assert plans[0] == [("a", 0, 8, True)]
    assert plans[1] == [("a", 8, 1, True), ("b", 0, 1, True)]
    assert len(a.generated) == 2 and len(b.generated) == 3


def test_max_batch_and_first_come_first_served():
    s = mk(max_batch=2, budget=64)
    reqs = [Request(i, [1] * 10, max_new=3 + i) for i in range(4)]
    for r in reqs:
        s.add(r)
    plans = drive(s)
    for p in plans:
        assert len(p) <= 2
    first_seen = {}
    for i, p in enumerate(plans):
        for rid, *_ in p:
            first_seen.setdefault(rid, i)
    assert first_seen[0] == first_seen[1] == 0 and first_seen[2] <= first_seen[3]
    assert first_seen[2] == 3  # as soon as request 0 (3 new tokens) has ended


def test_abort_gives_pages_and_slot_back():
    """A running request and a waiting one are ended from outside: pages and
    slot return, the others go on undisturbed."""
    s = mk(cache_pages=16, max_batch=2, budget=64)
    reqs = [Request(i, list(range(20)), max_new=6) for i in range(3)]
    for r in reqs:
        s.add(r)
    plan = s.plan()  # requests 0 and 1 run, 2 waits
    for e in plan:
        s.cache.advance(e.request.rid, e.n)
    s.commit(plan, [fake_token(e.request, e.start + e.n) for e in plan if e.wants_logits])
    assert s.abort(0) and s.abort(2) and not s.abort(99)
    assert [r.finish_reason for r in reqs] == ["aborted", None, "aborted"]
    assert [r.rid for r in s.finished] == [0, 2] and s.cache.live_requests() == [1]
    s.cache.check()
    drive(s)
    assert reqs[1].finish_reason == "length" and len(reqs[1].generated) == 6
    assert s.cache.live_requests() == [] and s.cache.free_pages() == 16 and s.cache.free_slots() == 2


def test_stop_ids_and_caps():
    s = mk(max_seq=20)
    r = Request("a", [1, 2, 3], max_new=50)
    stop_at = fake_token(r, 3 + 4)
    r.stop_ids = (stop_at,)
    s.add(r)
    drive(s)
    assert r.finish_reason == "stop" and r.generated[-1] == stop_at and len(r.generated) <= 5
    r2 = Request("b", [1, 2, 3], max_new=50)
    s.add(r2)
    drive(s)
    assert r2.finish_reason == "max_seq" and r2.n_known() == 20
    with pytest.raises(ValueError, match="can never fit"):
        s.add(Request("c", [0] * 20, 1))
    with pytest.raises(ValueError, match="empty prompt"):
        s.add(Request("d", [], 1))


def test_out_of_pages_preempts_the_youngest_and_recomputes():
    # 6 pages of 16: three requests of 30 tokens fill them; growing needs a 7th page
    s = mk(cache_pages=6, max_batch=3, budget=64)
    reqs = [Request(i, [i] * 30, max_new=8) for i in range(3)]
    for r in reqs:
        s.add(r)
    plans = drive(s)
    assert s.n_preemptions >= 1
    assert reqs[2].preemptions >= 1 and reqs[0].preemptions == 0  # the youngest gives way, the oldest never
    # the preempted request is fed again from its first token, generated tokens included
    refeeds = [p for plan in plans for p in plan if p[0] == 2 and p[1] == 0]
    assert len(refeeds) == 1 + reqs[2].preemptions
    for r in reqs:
        assert r.generated == [fake_token(r, 30 + i) for i in range(8)]  # same tokens as without preemption
    assert s.cache.free_pages() == 6


def test_alone_and_out_of_pages_ends_with_cache_full():
    s = mk(cache_pages=2, max_batch=1, budget=64, max_seq=1000)
    r = Request("a", [1] * 20, max_new=100, truncate=True)
    s.add(r)
    drive(s)
    assert r.finish_reason in ("cache_full", "max_seq") and r.n_known() <= 32


def test_waiting_request_is_not_admitted_without_room_for_its_prompt():
    s = mk(cache_pages=4, max_batch=4, budget=64)
    a, b = Request("a", [1] * 40, 4), Request("b", [2] * 40, 4)
    s.add(a), s.add(b)
    plans = drive(s)
    assert [p[0] for p in plans[0]] == ["a"]  # b's 41 tokens need 3 pages, 1 is free
    assert b.preemptions == 0 and len(b.generated) == 4


@pytest.mark.parametrize("seed", range(5))
def test_random_load_finishes_with_the_right_tokens(seed):
    rng = random.Random(seed)
    s = mk(cache_pages=rng.choice([8, 12, 40]), page=16, max_batch=rng.choice([2, 4, 8]), budget=rng.choice([8, 24, 100]))
    s.cache.n_slots  # noqa: B018
    reqs = [Request(i, [rng.randrange(50) for _ in range(rng.choice([1, 3, 20, 45, 90]))], max_new=rng.choice([1, 5, 30]))
            for i in range(12)]
    for r in reqs:
        s.add(r)
    drive(s)
    for r in reqs:
        assert r.finish_reason == "length" and r.generated == [fake_token(r, len(r.prompt) + i) for i in range(r.max_new)]


def test_decode_runs_between_host_checks():
    """Several decode steps in a row without the host seeing a token (the
    reference's sync_freq): only when every request decodes, nobody waits,
    and caps and pages allow it; a stop id inside the run ends the request
    there and drops what it sampled afterwards."""
    s = mk(cache_pages=64, max_batch=4, budget=64)
    a, b = Request("a", [1] * 10, max_new=25), Request("b", [2] * 3, max_new=7)
    s.add(a), s.add(b)
    assert s.plan_decode_run(10) == 0  # prompts not fed yet
    plan = s.plan()
    for e in plan:
        s.cache.advance(e.request.rid, e.n)
    s.commit(plan, [50, 60])
    assert s.plan_decode_run(10) == 6  # b may take 6 more tokens
    assert s.plan_decode_run(1) == 0
    s.add(Request("c", [3], max_new=2))
    assert s.plan_decode_run(10) == 0  # somebody waits for admission
    s.waiting.clear()
    n = s.plan_decode_run(4)
    assert n == 4
    for r in (a, b):
        s.cache.reserve(r.rid, n)
        s.cache.advance(r.rid, n)
    a.stop_ids = (77,)
    done = s.commit_run([[70, 80], [77, 81], [72, 82], [73, 83]])
    assert done == [a] and a.finish_reason == "stop" and a.generated == [50, 70, 77]
    assert b.generated == [60, 80, 81, 82, 83] and b.n_fed == 3 + 4 and b.remaining() == 1
    assert s.plan_decode_run(10) == 2  # b: 7 - 5
    s.cache.reserve("b", 2), s.cache.advance("b", 2)
    assert s.commit_run([[90], [91]]) == [b] and b.finish_reason == "length" and len(b.generated) == 7
    assert s.cache.free_pages() == 64
    # pages: a run must fit for all requests at once
    for pages, want in ((4, 10), (3, 0)):
        t = mk(cache_pages=pages, max_batch=2, budget=64)
        rs = [Request(i, [1] * 15, max_new=40, truncate=True) for i in range(2)]
        for r in rs:
            t.add(r)
        plan = t.plan()
        for e in plan:
            t.cache.advance(e.request.rid, e.n)
        t.commit(plan, [5, 6])  # both hold 15 tokens in one page; the 17th token needs a second page each
        assert t.plan_decode_run(10) == want
    # the cap of one request's length (here the pool itself) bounds a run
    t = mk(cache_pages=2, max_batch=1, budget=64)
    r = Request("r", [1] * 28, max_new=50, truncate=True)
    t.add(r)
    plan = t.plan()
    t.cache.advance("r", 28)
    t.commit(plan, [5])
    assert t.plan_decode_run(10) == 3


# ----------------------------------------------- the host one step behind
def drive_one_step_behind(sched, max_steps=10_000):
    """As :func:`drive`, but a step's tokens reach the scheduler only after the next step is planned
    and committed (the engine's overlapped steps): ``commit`` without tokens, ``resolve`` a step later."""
    from fastgen_amd.engine.scheduler import PENDING

    in_flight = None
    reported = []
    for _ in range(max_steps):
        reported += [r.rid for r in sched.finished]
        sched.finished.clear()
        if not sched.has_work() and in_flight is None:
            break
        plan = sched.plan()
        if plan:
            assert sum(e.n for e in plan) <= sched.max_step_tokens
            for e in plan:
                assert e.request.finish_reason is None, "a request that has ended runs again"
                assert e.start == e.request.n_fed == sched.cache.length(e.request.rid)
                toks = e.request.tokens_from(e.start, e.n)
                assert PENDING not in toks or (e.n == 1 and in_flight is not None and
                                               any(p.request is e.request and p.wants_logits for p in in_flight[0]))
                sched.cache.advance(e.request.rid, e.n)
            sched.cache.check()
            tokens = [fake_token(e.request, e.start + e.n) for e in plan if e.wants_logits]
            sched.commit(plan)  # the tokens are "still on the device"
        if in_flight is not None:
            sched.resolve(*in_flight)
            in_flight = None
        if plan:
            in_flight = (plan, tokens)
    else:
        raise AssertionError("the scheduler did not finish")
    return reported


@pytest.mark.parametrize("admit_reserve", [0, 16, 128])
@pytest.mark.parametrize("seed", range(16))
def test_one_step_behind_gives_the_same_requests(seed, admit_reserve):
    """Random loads with stop ids, small budgets and few pages (preemption): every request ends with the
    same tokens and for the same reason whether the scheduler sees a step's tokens at once or a step
    late; nothing is left pending, no page is lost."""
    def load():
        rng = random.Random(100 + seed)
        # odd seeds: pools so tight that decoding requests are preempted with a sample still pending
        pages = rng.choice([8, 12, 40]) if seed % 2 == 0 else rng.choice([7, 8, 9])
        s = mk(cache_pages=pages, page=16, max_batch=rng.choice([2, 4, 8]),
               budget=rng.choice([8, 24, 100]), max_seq=rng.choice([None, 60]), admit_reserve=admit_reserve)
        reqs = []
        for i in range(14):
            n = rng.choice([1, 3, 20, 45, 90]) if seed % 2 == 0 else rng.choice([7, 15, 30, 31, 47])
            if s.max_seq <= n:
                n = 3
            r = Request(i, [rng.randrange(50) for _ in range(n)], max_new=rng.choice([1, 5, 30]), truncate=True)
            if rng.random() < 0.5:  # a stop id that the stand-in model samples at some step, or never
                r.stop_ids = (fake_token(r, n + rng.randrange(0, 12)), 2)
            reqs.append(r)
            s.add(r)
        return s, reqs

    s1, reqs1 = load()
    drive(s1)
    s2, reqs2 = load()
    reported = drive_one_step_behind(s2)
    assert sorted(reported) == list(range(14))  # every request is reported as ended exactly once
    for a, b in zip(reqs1, reqs2):
        assert b.n_pending == 0 and -1 not in b.generated
        assert (a.generated, a.finish_reason) == (b.generated, b.finish_reason), a.rid
    assert s2.cache.live_requests() == [] and s2.cache.free_pages() == s1.cache.free_pages()
    s2.cache.check()


@pytest.mark.parametrize("admit_reserve", [0, 16, 128])
@pytest.mark.parametrize("seed", range(8))
def test_aborts_at_any_time_lose_nothing(seed, admit_reserve):
    """Requests are aborted at random moments (waiting, mid-prompt, decoding with a sample still pending,
    preempted) while the scheduler runs a step behind: every request is reported exactly once, an aborted one
    never runs again, its late sample is still filled in, and every page and slot comes back."""
    from fastgen_amd.engine.scheduler import PENDING

    rng = random.Random(500 + seed)
    pages = rng.choice([7, 9, 40])
    s = mk(cache_pages=pages, page=16, max_batch=rng.choice([2, 4]), budget=rng.choice([8, 24, 100]),
           admit_reserve=admit_reserve)
    reqs = [Request(i, [rng.randrange(50) for _ in range(rng.choice([1, 7, 30, 47]))], max_new=rng.choice([1, 5, 30]),
                    truncate=True) for i in range(12)]
    for r in reqs:
        s.add(r)
    in_flight, reported, aborted = None, [], set()
    for _ in range(10_000):
        reported += [r.rid for r in s.finished]
        s.finished.clear()
        if not s.has_work() and in_flight is None:
            break
        if rng.random() < 0.3:
            victim = rng.choice(reqs)
            if victim.finish_reason is None:
                assert s.abort(victim.rid)
                aborted.add(victim.rid)
            else:
                assert not s.abort(victim.rid)  # ended already: nothing to abort
        plan = s.plan()
        if plan:
            for e in plan:
                assert e.request.rid not in aborted and e.request.finish_reason is None
                s.cache.advance(e.request.rid, e.n)
            s.cache.check()
            tokens = [fake_token(e.request, e.start + e.n) for e in plan if e.wants_logits]
            s.commit(plan)
        if in_flight is not None:
            s.resolve(*in_flight)
            in_flight = None
        if plan:
            in_flight = (plan, tokens)
    else:
        raise AssertionError("the scheduler did not finish")
    assert sorted(reported) == list(range(12))
    for r in reqs:
        assert r.n_pending == 0 and PENDING not in r.generated
        assert (r.finish_reason == "aborted") == (r.rid in aborted)
    assert s.cache.live_requests() == [] and s.cache.free_pages() == pages and s.cache.free_slots() == s.max_batch
    s.cache.check()


def test_a_stop_id_seen_a_step_late_drops_the_step_after_it():
    from fastgen_amd.engine.scheduler import PENDING

    s = mk()
    r = Request("a", [1, 2, 3], max_new=10, stop_ids=(77,), want_logprobs=True)
    s.add(r)
    p0 = s.plan()
    s.cache.advance("a", 3)
    assert s.commit(p0) == [] and r.generated == [PENDING] and r.n_pending == 1
    p1 = s.plan()  # planned from the count alone: one token, value unknown
    assert [(e.start, e.n, e.wants_logits) for e in p1] == [(3, 1, True)] and r.tokens_from(3, 1) == [PENDING]
    s.cache.advance("a", 1)
    s.commit(p1)
    assert r.generated == [PENDING, PENDING]
    assert s.resolve(p0, [77], [-0.5]) == [r]  # the first token was a stop id
    assert r.generated == [77] and r.logprobs == [-0.5] and r.finish_reason == "stop" and r.n_pending == 0
    assert not s.has_work() and s.cache.live_requests() == []
    assert s.resolve(p1, [5], [-1.0]) == [] and r.generated == [77]  # what the step after it sampled is dropped
    # a request that its token count ended: the stop id found later is the reason
    q = Request("b", [1], max_new=1, stop_ids=(9,))
    s.add(q)
    p = s.plan()
    s.cache.advance("b", 1)
    assert s.commit(p) == [q] and q.finish_reason == "length"
    s.resolve(p, [9])
    assert q.finish_reason == "stop" and q.generated == [9]


def test_a_late_stop_id_of_a_preempted_request_ends_it_once():
    """A decoding request is preempted while its last sample is still on the device; the sample
    turns out to be a stop id.  The request ends there: it is in neither line, is reported once,
    and is never admitted again."""
    s = mk(cache_pages=2, page=8, max_batch=2, budget=64)
    a, b = Request("a", [1] * 7, max_new=8, stop_ids=(99,)), Request("b", [2] * 7, max_new=8, stop_ids=(99,))
    s.add(a), s.add(b)
    p0 = s.plan()
    assert [(e.request.rid, e.n) for e in p0] == [("a", 7), ("b", 7)]
    for e in p0:
        s.cache.advance(e.request.rid, e.n)
    assert s.commit(p0) == []  # both samples pending
    p1 = s.plan()  # a and b decode: the 8th token still fits each one's page
    for e in p1:
        s.cache.advance(e.request.rid, e.n)
    s.commit(p1)
    s.resolve(p0, [7, 6])
    p2 = s.plan()  # the 9th token of a needs a page: b, the youngest, gives way with a sample pending
    assert [e.request.rid for e in p2] == ["a"] and b.preemptions == 1 and b.n_pending == 1
    assert any(r is b for r in s.waiting)
    s.cache.advance("a", 1)
    s.commit(p2)
    late = s.resolve(p1, [8, 99])  # b's pending token is a stop id
    assert late == [b] and b.finish_reason == "stop" and b.generated == [6, 99]
    assert not any(r is b for r in s.waiting) and not any(r is b for r in s.running)
    assert [r.rid for r in s.finished].count("b") == 1
    s.finished.clear()
    s.resolve(p2, [9])
    reported = drive_one_step_behind(s)
    assert "b" not in reported and b.generated == [6, 99] and a.finish_reason == "length"
    assert s.cache.live_requests() == [] and s.cache.free_pages() == 2


def test_a_request_that_can_never_fit_is_refused_unless_it_agrees_to_be_cut():
    s = mk(cache_pages=4, page=16, max_batch=2, budget=64)  # 64 tokens of cache
    with pytest.raises(ValueError, match="can never fit.*holds 64 tokens"):
        s.add(Request("a", [1] * 40, max_new=25))
    assert not s.has_work()
    s.add(Request("b", [1] * 40, max_new=24))  # 64 exactly: fits
    r = Request("c", [1] * 40, max_new=100, truncate=True)
    s.add(r)
    drive(s)
    assert r.finish_reason == "max_seq" and r.n_known() == 64


def test_a_budget_smaller_than_the_decoding_requests_goes_round():
    """max_step_tokens < live decoders: every request advances, none is left out of every step."""
    s = mk(cache_pages=64, page=16, max_batch=5, budget=5)
    reqs = [Request(i, [i + 1], max_new=12) for i in range(5)]
    for r in reqs:
        s.add(r)
    plan = s.plan()  # all five prompts
    for e in plan:
        s.cache.advance(e.request.rid, e.n)
    s.commit(plan, [5] * 5)
    s.max_step_tokens = 2
    served = {r.rid: 0 for r in reqs}
    for _ in range(10):
        plan = s.plan()
        assert sum(e.n for e in plan) <= 2
        for e in plan:
            served[e.request.rid] += 1
            s.cache.advance(e.request.rid, e.n)
        s.commit(plan, [5] * sum(e.wants_logits for e in plan))
    assert max(served.values()) - min(served.values()) <= 1, served
    drive(s)
    assert all(len(r.generated) == 12 for r in reqs)


def test_admission_keeps_room_for_what_running_requests_will_generate():
    """The reference asks for the prompt and a 128-token buffer when it admits a request
    (fastgen/generate.py:535-536): requests that generate no more than the reserve never have to
    give way.  The same load with and without the reserve: same tokens, preemptions only without."""
    def load(reserve):
        s = mk(cache_pages=12, page=16, max_batch=8, budget=256, admit_reserve=reserve)
        reqs = [Request(i, [i] * 30, max_new=30) for i in range(6)]  # 60 tokens = 4 pages each at the end
        for r in reqs:
            s.add(r)
        return s, reqs

    s0, r0 = load(0)
    plans0 = drive(s0)
    assert len(plans0[0]) == 6 and s0.n_preemptions > 0  # all admitted at once: 12 pages; they need 24
    s1, r1 = load(128)
    plans1 = drive(s1)
    assert s1.n_preemptions == 0
    assert len(plans1[0]) == 3  # three requests of 4 pages each fill the 12 pages
    for a, b in zip(r0, r1):
        assert a.generated == b.generated and b.finish_reason == "length"
    # the reserve is a horizon, not a promise of everything: requests that generate far more than it
    # are admitted beyond what they will need in the end (and may give way later)
    s2 = mk(cache_pages=12, page=16, max_batch=8, budget=256, admit_reserve=16)
    for i in range(6):
        s2.add(Request(i, [i] * 30, max_new=100, truncate=True))
    assert len(s2.plan()) == 4  # 46 tokens = 3 pages each
    # a request alone is admitted as soon as its prompt fits, whatever the reserve
    s3 = mk(cache_pages=2, page=16, max_batch=2, budget=64, admit_reserve=128)
    s3.add(Request("a", [1] * 20, max_new=12))
    assert [e.request.rid for e in s3.plan()] == ["a"]


def test_memory_budget_counts_the_per_request_state():
    """The cache's size from a memory budget: pages take what the reserve and the per-request state
    tensors (one row a slot, and one more) leave."""
    import torch

    from fastgen_amd.cache.storage import bytes_per_token, group_entries, state_bytes, tokens_that_fit
    from fastgen_amd.parts import PagedNeed, StateNeed

    groups = group_entries([PagedNeed(2, 16, None), PagedNeed(2, 16, None), None, PagedNeed(1, 32, 64)])
    per_token = bytes_per_token(groups, torch.bfloat16)
    assert per_token == 2 * 2 * 32 * 2 + 1 * 64 * 2
    needs = {2: StateNeed((100, 8), torch.float32), 3: StateNeed((7,), torch.bfloat16)}
    assert state_bytes(needs, 9) == 10 * (100 * 8 * 4 + 7 * 2)
    assert state_bytes({}, 9) == 0
    free, reserve, page = 10_000_000, 1_000_000, 16
    plain = tokens_that_fit(free, groups, page, torch.bfloat16, reserve)
    assert plain == (free - reserve) // per_token // page * page
    with_state = tokens_that_fit(free, groups, page, torch.bfloat16, reserve, needs, 999)
    assert with_state == (free - reserve - state_bytes(needs, 999)) // per_token // page * page < plain
    # the pools and the state together stay inside the budget
    assert with_state * per_token + state_bytes(needs, 999) + reserve <= free
    assert tokens_that_fit(free, groups, page, torch.bfloat16, reserve, needs, 999, at_most=100) == 96
    assert tokens_that_fit(free, groups, page, torch.bfloat16, reserve, needs, 10 ** 6) == 0  # the state alone is too much


def test_step_memory_estimate_sees_the_widest_product():
    """What a step's intermediate tensors may take is sized by the widest matrix of a layer (here the
    gate/up matrix, 2 x 192 rows), whatever the part keeps its matrices in."""
    import torch

    from fastgen_amd.engine import Model
    from fastgen_amd.engine.engine import step_memory_estimate
    from plain_llama import TINY_A

    model = Model.random(TINY_A, 0, torch.float32, "cpu")
    widest = 2 * TINY_A["intermediate_size"]
    assert widest > TINY_A["hidden_size"]
    assert step_memory_estimate(model, 100, 4) == 100 * 12 * widest + 3 * 4 * TINY_A["vocab_size"] * 4
