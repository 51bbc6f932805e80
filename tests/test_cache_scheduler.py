"""The cache manager and the scheduler's decisions, without a GPU: pages are never lost, held
twice or freed twice under random orders of requests; window groups give pages back; admission,
token budget, portions, preemption and failure are decided as documented."""
import random

import pytest
import torch

from infinilm_amd.cache import CacheError, CacheManager, FixedState, OutOfPages, PagedKV, PagePool
from infinilm_amd.engine.request import FinishReason, InferenceRequest, RequestStatus
from infinilm_amd.engine.scheduler import Scheduler
from infinilm_amd.sampling import SamplingParams


def _cache(num_pages=8, page_size=4, needs=None, max_requests=6):
    needs = needs if needs is not None else [PagedKV(1, 4), PagedKV(1, 4)]
    return CacheManager(needs, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                        dtype=torch.float32, device="cpu")


def test_page_pool_fifo_and_errors():
    pool = PagePool(4)
    a = pool.take(3)
    assert a == [0, 1, 2] and pool.num_free == 1
    with pytest.raises(OutOfPages):
        pool.take(2)
    assert pool.num_free == 1  # nothing taken by the failed call
    pool.give_back([1])
    assert pool.take(2) == [3, 1]  # first freed, first reused, after what was already free
    with pytest.raises(CacheError, match="twice"):
        pool.give_back([0, 0])
    with pytest.raises(CacheError, match="not of this pool"):
        pool.give_back([9])
    pool.check()
    assert pool.high_water == 4


def test_slots_pages_and_block_tables():
    c = _cache(num_pages=5, page_size=4)
    c.admit("a")
    c.reserve("a", 6)
    assert c.table("a", 0) == [0, 1] and c.pages_needed("a", 6) == [0]
    c.commit("a", 6)
    # slot = page * page_size + offset (cache_manager.py:186-191)
    assert [c.slot_of("a", 0, p) for p in (0, 3, 4, 5)] == [0, 3, 4, 5]
    assert c.pages_needed("a", 2) == [0] and c.pages_needed("a", 3) == [1]   # a new page iff a token opens one
    c.admit("b")
    c.reserve("b", 9)
    assert c.table("b", 0) == [2, 3, 4] and c.free_pages() == 0
    with pytest.raises(OutOfPages):
        c.reserve("a", 3)
    assert c.table("a", 0) == [0, 1]
    c.reserve("a", 2)
    c.commit("a", 2)
    with pytest.raises(CacheError, match="beyond what was reserved"):
        c.commit("a", 1)
    c.release("b")
    assert c.free_pages() == 3
    c.reserve("a", 3)
    assert c.table("a", 0) == [0, 1, 2]   # b's first page is reused first
    with pytest.raises(CacheError, match="released twice"):
        c.release("b")
    with pytest.raises(CacheError, match="already admitted"):
        c.admit("a")
    c.check()
    c.release("a")
    assert c.free_pages() == 5


def test_window_group_has_pages_of_its_own_and_gives_them_back():
    c = _cache(num_pages=6, page_size=4, needs=[PagedKV(1, 4), PagedKV(1, 4, window=6), PagedKV(2, 8)])
    assert len(c.groups) == 2 and c.group_of_entry == {0: 0, 1: 1, 2: 0}
    assert c.k[2].shape == (6 + 1, 2, 4, 8) and c.null_page(0) == 6   # one page more: for rows of no request
    c.admit("a")
    for n in (5, 1, 1, 4, 1):
        c.reserve("a", n)
        c.commit("a", n)
    # 12 tokens cached: the next query (position 12) sees keys 7..12 -> logical pages 1.. are needed
    assert c.table("a", 0) == [0, 1, 2]
    assert c.table("a", 1)[0] == -1 and all(p >= 0 for p in c.table("a", 1)[1:])
    assert c.groups[1].pool.num_free == 6 - 2 and c.groups[0].pool.num_free == 3
    with pytest.raises(CacheError, match="already given back"):
        c.slot_of("a", 1, 2)
    c.check()
    c.release("a")
    assert c.groups[0].pool.num_free == 6 and c.groups[1].pool.num_free == 6


def test_state_slots():
    c = _cache(needs=[PagedKV(1, 4), FixedState((3, 2))], max_requests=2)
    assert c.state[1].shape == (2 + 2, 3, 2) and not c.state[1].any() and c.null_state_row == 3   # zero row, 2 slots, row of no request
    c.admit("a")
    c.admit("b")
    ra, rb = c.state_rows("a"), c.state_rows("b")
    assert ra[0] == 0 and rb[0] == 0 and {ra[1], rb[1]} == {1, 2}   # fresh: read the zero row
    c.reserve("a", 2)
    c.commit("a", 2)
    assert c.state_rows("a") == (ra[1], ra[1])
    with pytest.raises(CacheError, match="no state slot"):
        c.admit("c")
    c.release("a")
    c.admit("c")
    assert c.state_rows("c") == (0, ra[1])
    c.check()
    # a step that runs twice on the same books (the warm-up before a graph is recorded) puts the rows back
    c.state[1][rb[1]] = 5.0
    saved = c.snapshot_states(["b"])
    c.state[1][rb[1]] += 1.0
    c.state[1][ra[1]] = 9.0          # another request's row is not touched by the restore
    c.restore_states(saved)
    assert float(c.state[1][rb[1]].min()) == 5.0 == float(c.state[1][rb[1]].max()) and float(c.state[1][ra[1]].max()) == 9.0
    assert _cache(needs=[PagedKV(1, 4)], max_requests=2).snapshot_states([]) == []


@pytest.mark.parametrize("seed", range(6))
def test_no_page_lost_held_twice_or_freed_twice_under_random_orders(seed):
    rng = random.Random(seed)
    c = _cache(num_pages=24, page_size=4, needs=[PagedKV(1, 4), PagedKV(1, 4, window=10)], max_requests=5)
    live = {}
    n_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.2 and len(live) < 5:
            rid = f"r{n_id}"
            n_id += 1
            c.admit(rid)
            live[rid] = 0
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 11])
            if c.can_reserve(rid, n):
                c.reserve(rid, n)
                c.commit(rid, n)
                live[rid] += n
                assert c.length(rid) == live[rid]
            else:
                before = [g.pool.num_free for g in c.groups]
                with pytest.raises(OutOfPages):
                    c.reserve(rid, n)
                assert before == [g.pool.num_free for g in c.groups]
        elif live:
            rid = rng.choice(list(live))
            c.release(rid)
            del live[rid]
        c.check()
        for rid, n in live.items():   # the pages a request needs for its window and its length are held
            t0, t1 = c.table(rid, 0), c.table(rid, 1)
            assert len(t0) >= -(-n // 4) and all(p >= 0 for p in t0)
            lo = max(0, n - 10 + 1) // 4
            assert all(p >= 0 for p in t1[lo:]) and all(p == -1 for p in t1[:lo])
    for rid in list(live):
        c.release(rid)
    assert all(g.pool.num_free == 24 for g in c.groups)


def test_published_pages_are_shared_idle_and_taken_last():
    pool = PagePool(4)
    a, b = pool.take(2)
    assert pool.publish(a, b"k1") and pool.publish(b, b"k2") and pool.lookup(b"k1") == a
    with pytest.raises(CacheError, match="published twice"):
        pool.publish(a, b"k3")
    c = pool.take(1)[0]
    assert not pool.publish(c, b"k1") and not pool.is_published(c)     # the same content is there already
    pool.share(a)
    assert pool.refs(a) == 2
    with pytest.raises(CacheError, match="not published"):
        pool.share(c)
    pool.give_back([b, a])                 # b idle, a still held once
    assert pool.num_idle == 1 and pool.num_free == 2 and pool.lookup(b"k2") == b
    pool.give_back([a])
    assert pool.num_idle == 2 and pool.num_held == 1
    pool.check()
    pool.share(b)                          # an idle page found again is held again
    assert pool.num_idle == 1 and pool.refs(b) == 1
    got = pool.take(2)                     # the free page first, then the idle one, which loses its content
    assert got == [3, a] and pool.lookup(b"k1") is None and pool.evictions == 1 and not pool.is_published(a)
    with pytest.raises(OutOfPages):
        pool.take(1)
    pool.give_back([got[0]])
    with pytest.raises(CacheError, match="nobody holds"):
        pool.publish(got[0], b"x")
    pool.check()


def _shared_cache(num_pages=10, page_size=4, **kw):
    return CacheManager([PagedKV(1, 4), PagedKV(2, 8)], page_size=page_size, num_pages=num_pages, max_requests=6,
                        dtype=torch.float32, device="cpu", prefix_caching=True, **kw)


def test_a_request_takes_over_the_published_pages_of_its_beginning():
    c = _shared_cache()
    assert c.prefix_caching
    toks = list(range(100, 111))            # 11 tokens: two whole pages and three
    assert c.admit("a", toks) == 0 and c.peek_prefix(toks) == (0, 0)
    c.reserve("a", 11)
    c.commit("a", 6, toks[:6])              # one whole page computed
    assert c.peek_prefix(toks) == (4, 0)
    c.commit("a", 5, toks[6:])
    assert c.peek_prefix(toks) == (8, 0) and c.table("a", 0) == [0, 1, 2]
    # the same beginning: the whole pages are shared, the rest is the request's own
    assert c.admit("b", toks[:8] + [7, 7, 7]) == 8
    assert c.table("b", 0) == [0, 1] and c.length("b") == 8 and c.pages_needed("b", 3) == [1]
    c.reserve("b", 3)
    assert c.table("b", 0) == [0, 1, 3]
    c.check()
    # never the page of the last token: a prompt of exactly two pages takes one over
    assert c.peek_prefix(toks[:8]) == (4, 0) and c.peek_prefix(toks[:9]) == (8, 0) and c.peek_prefix(toks[:4]) == (0, 0)
    # another beginning finds nothing, and a page is only found behind the pages before it
    assert c.peek_prefix([1] + toks[1:]) == (0, 0) and c.peek_prefix([9, 9, 9, 9] + toks[4:]) == (0, 0)
    c.release("a")                          # its shared pages stay held by b, its own last page is free again
    assert c.free_pages() == 10 - 3 and c.groups[0].pool.num_idle == 0
    c.release("b")
    assert c.free_pages() == 10 and c.groups[0].pool.num_idle == 2
    assert c.peek_prefix(toks) == (8, 2)    # still findable, and idle
    assert c.admit("c", toks) == 8 and c.groups[0].pool.num_idle == 0
    st = c.stats()
    assert st["prefix_hit_tokens"] == 16 and st["prefix_asked_tokens"] == 33
    c.release("c")
    c.check()


def test_idle_pages_give_way_from_the_end_of_a_run():
    c = _shared_cache(num_pages=4)
    toks = list(range(13))
    c.admit("a", toks)
    c.reserve("a", 13)
    c.commit("a", 13, toks)
    c.release("a")                          # three published pages idle, one free
    assert c.groups[0].pool.num_idle == 3 and c.free_pages() == 4
    c.admit("x")
    c.reserve("x", 8)                       # the free page, then the end of a's run
    assert c.peek_prefix(toks) == (8, 2)
    c.commit("x", 8)                        # committed without tokens: nothing of x is ever published
    c.reserve("x", 4)
    assert c.peek_prefix(toks) == (4, 1)
    c.check()
    c.commit("x", 4)
    c.release("x")
    assert c.groups[0].pool.num_idle == 1 and c.free_pages() == 4
    # a request whose tokens stop being told stops publishing, and says so by never being found
    c.admit("y", [5] * 9)
    c.reserve("y", 9)
    c.commit("y", 4, [5] * 4)
    c.commit("y", 5)
    assert c.peek_prefix([5] * 9) == (4, 0)
    c.release("y")
    c.check()


def test_prefix_sharing_is_off_where_a_window_or_a_state_is_kept():
    w = CacheManager([PagedKV(1, 4), PagedKV(1, 4, window=8)], page_size=4, num_pages=8, max_requests=2,
                     dtype=torch.float32, device="cpu", prefix_caching=True)
    s = CacheManager([PagedKV(1, 4), FixedState((3,))], page_size=4, num_pages=8, max_requests=2,
                     dtype=torch.float32, device="cpu", prefix_caching=True)
    for c in (w, s):
        assert not c.prefix_caching
        assert c.admit("a", list(range(9))) == 0
        c.reserve("a", 9)
        c.commit("a", 9, list(range(9)))
        assert c.peek_prefix(list(range(9))) == (0, 0)
        c.release("a")
        assert c.groups[0].pool.num_idle == 0


@pytest.mark.parametrize("seed", range(4))
def test_shared_pages_under_random_orders(seed):
    """Requests drawn from a few prompts that share beginnings, admitted, advanced and released in
    random order with few pages: owners and block tables agree at every moment, what is found under
    a request's tokens are its own published pages, nothing is lost at the end."""
    rng = random.Random(100 + seed)
    c = _shared_cache(num_pages=14, page_size=4)
    stems = [[rng.randrange(50) for _ in range(20)] for _ in range(2)]
    live = {}
    n_id = 0
    for _ in range(700):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            stem = rng.choice(stems)
            toks = stem[:rng.randrange(1, 21)] + [rng.randrange(50) for _ in range(rng.randrange(0, 8))]
            rid = f"r{n_id}"
            n_id += 1
            want, idle = c.peek_prefix(toks)
            free_before = c.free_pages()
            got = c.admit(rid, toks)
            assert got == want and got <= len(toks) - 1 and got % 4 == 0 and c.free_pages() == free_before - idle
            live[rid] = (toks, got)
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            toks, done = live[rid]
            n = min(rng.choice([1, 1, 2, 5, 11]), len(toks) - done)
            if n == 0:                      # the prompt is through: a generated token
                toks.append(rng.randrange(50))
                n = 1
            if c.can_reserve(rid, n):
                c.reserve(rid, n)
                c.commit(rid, n, toks[done:done + n])
                live[rid] = (toks, done + n)
                assert c.length(rid) == done + n
        elif live:
            rid = rng.choice(list(live))
            c.release(rid)
            del live[rid]
        c.check()
        for rid, (toks, done) in live.items():
            # what is findable under a live request's tokens never exceeds its whole pages, and where its
            # own pages are the published ones they are what is found
            pages, _ = c._matching_pages(toks[:done] + [0])
            assert len(pages) <= done // 4
            own = c.table(rid, 0)
            assert all(p == own[i] for i, p in enumerate(pages) if c.groups[0].pool.is_published(own[i]))
    for rid in list(live):
        c.release(rid)
    c.check()
    assert c.free_pages() == 14 and not c.requests


# ------------------------------------------------------------------------------------------------
# scheduler
# ------------------------------------------------------------------------------------------------
def _req(rid, n_prompt, max_tokens=4, **kw):
    return InferenceRequest(rid, list(range(1, n_prompt + 1)), SamplingParams(max_tokens=max_tokens, **kw),
                            eos_token_ids=[99], key=hash(rid) & 0xffff)


def _run(sched, token_of=lambda req: 7, max_steps=500):
    """The engine loop with a step function that samples fixed tokens; the cache is advanced as
    the real step function advances it."""
    steps = []
    for _ in range(max_steps):
        if not sched.has_unfinished():
            break
        out = sched.schedule()
        assert out.entries, "the scheduler made no progress"
        for e in out.entries:
            assert e.start == sched.cache.length(e.request.request_id)
            sched.cache.reserve(e.request.request_id, e.num_tokens)
            sched.cache.commit(e.request.request_id, e.num_tokens, e.request.token_slice(e.start, e.num_tokens))
        sched.update(out, {e.request.request_id: token_of(e.request) for e in out.entries if e.samples})
        sched.cache.check()
        steps.append(out)
    assert not sched.has_unfinished()
    return steps


def test_portions_under_a_token_budget_and_mixed_steps():
    c = _cache(num_pages=64, page_size=4)
    s = Scheduler(c, max_num_seqs=4, max_num_batched_tokens=10, chunk_size=8, max_positions=1000)
    a, b = _req("a", 19, max_tokens=3), _req("b", 5, max_tokens=6)
    s.add_request(a)
    s.add_request(b)
    steps = _run(s)
    shape = [[(e.request.request_id, e.start, e.num_tokens, e.samples) for e in o.entries] for o in steps]
    assert shape[0] == [("a", 0, 8, False), ("b", 0, 2, False)]        # budget 10 = 8 + 2
    assert shape[1] == [("a", 8, 8, False), ("b", 2, 2, False)]
    assert shape[2] == [("a", 16, 3, True), ("b", 4, 1, True)]          # both prompts end here
    assert shape[3] == [("a", 19, 1, True), ("b", 5, 1, True)]          # decode beside decode
    assert all(o.num_tokens <= 10 for o in steps)
    assert a.finish_reason == FinishReason.LENGTH and a.output_token_ids == [7, 7, 7]
    assert b.get_num_generated_tokens() == 6 and c.free_pages() == 64
    # decodes come first in a step, portions of prompts fill the rest of the budget
    c2 = _cache(num_pages=64, page_size=4)
    s2 = Scheduler(c2, max_num_seqs=4, max_num_batched_tokens=6, max_positions=1000)
    s2.add_request(_req("x", 2, max_tokens=5))
    out = s2.schedule()
    for e in out.entries:
        c2.reserve("x", e.num_tokens); c2.commit("x", e.num_tokens)
    s2.update(out, {"x": 7})
    s2.add_request(_req("y", 20, max_tokens=2))
    out = s2.schedule()
    assert [(e.request.request_id, e.num_tokens) for e in out.entries] == [("x", 1), ("y", 5)]


def test_finish_reasons_and_freeing():
    c = _cache(num_pages=16, page_size=4)
    s = Scheduler(c, max_num_seqs=4, max_num_batched_tokens=64, max_positions=12)
    eos, stop, ign, pos = _req("eos", 3, 8), _req("stop", 3, 8, stop_token_ids=[55]), _req("ign", 3, 3, ignore_eos=True), _req("pos", 9, 50)
    for r in (eos, stop, ign, pos):
        s.add_request(r)
    toks = {"eos": [5, 99, 5], "stop": [55], "ign": [99, 99, 99], "pos": [1] * 50}
    _run(s, token_of=lambda r: toks[r.request_id][r.get_num_generated_tokens()])
    assert eos.finish_reason == FinishReason.EOS_TOKEN and eos.output_token_ids == [5, 99]
    assert stop.finish_reason == FinishReason.STOP
    assert ign.finish_reason == FinishReason.LENGTH and ign.output_token_ids == [99, 99, 99]
    assert pos.finish_reason == FinishReason.LENGTH and pos.num_known_tokens() == 12   # the position table ends
    assert c.free_pages() == 16 and all(r.status == RequestStatus.FINISHED for r in (eos, stop, ign, pos))


def test_rejections_at_add():
    c = _cache(num_pages=4, page_size=4)
    s = Scheduler(c, max_num_seqs=4, max_num_batched_tokens=64, max_positions=100)
    big, empty, long = _req("big", 16), _req("empty", 0), _req("long", 100)
    for r in (big, empty, long):
        s.add_request(r)
        assert r.status == RequestStatus.FAILED and r.finish_reason == FinishReason.ERROR
    assert "no_capacity" in big.error and not s.has_unfinished()
    s2 = Scheduler(_cache(num_pages=4, page_size=4), 4, 64, policy="reserve_full", max_positions=100)
    r = _req("r", 8, max_tokens=20)
    s2.add_request(r)
    assert r.status == RequestStatus.FAILED and "max_tokens" in r.error


def test_reserve_full_admission_never_runs_out_and_blocks_head_of_line():
    c = _cache(num_pages=8, page_size=4)
    s = Scheduler(c, max_num_seqs=8, max_num_batched_tokens=64, policy="reserve_full", max_positions=1000)
    reqs = [_req("a", 6, max_tokens=10), _req("b", 9, max_tokens=7), _req("c", 2, max_tokens=2), _req("d", 3, 5)]
    for r in reqs:
        s.add_request(r)
    out = s.schedule()
    # a needs 4 pages, b needs 4: the pool is promised; c would fit a page count but waits behind nothing free
    assert [e.request.request_id for e in out.entries] == ["a", "b"]
    for e in out.entries:
        c.reserve(e.request.request_id, e.num_tokens); c.commit(e.request.request_id, e.num_tokens)
    s.update(out, {"a": 7, "b": 7})
    steps = _run(s)
    assert s.num_preemptions == 0 and all(r.finish_reason == FinishReason.LENGTH for r in reqs)
    first_c = next(i for i, o in enumerate(steps) if any(e.request.request_id == "c" for e in o.entries))
    first_d = next(i for i, o in enumerate(steps) if any(e.request.request_id == "d" for e in o.entries))
    assert first_c <= first_d   # first come, first served
    assert c.free_pages() == 8


def test_reserve_full_counts_each_group_by_its_own_need():
    """Two groups: one keeps all keys, one a window of 6 keys.  Full reservation asks of each group what a request
    can hold there at most: all its pages in the first, the window's few in the second, so a small pool for the
    windowed layers does not hold back requests that would never fill it; and no step ever runs out of pages."""
    needs = [PagedKV(1, 4), PagedKV(1, 4, window=6)]
    c = CacheManager(needs, page_size=4, num_pages=16, max_requests=6, dtype=torch.float32, device="cpu",
                     num_pages_per_group={6: 9})
    s = Scheduler(c, max_num_seqs=4, max_num_batched_tokens=16, chunk_size=4, policy="reserve_full", max_positions=1000)
    assert s._group_pages(c.groups[0], 30) == 8 and s._group_pages(c.groups[1], 30) == 4   # window 6 + portion 4 -> 3 pages + 1
    reqs = [_req("a", 20, max_tokens=10), _req("b", 18, max_tokens=12), _req("c", 5, max_tokens=3)]
    for r in reqs:
        s.add_request(r)
    out = s.schedule()
    # all keys: a and b need 8 pages each of 16; c waits for them (head of line).  With one need for all groups, b (8 pages)
    # would not have fitted beside a in the windowed group's 9 pages.
    assert [e.request.request_id for e in out.entries] == ["a", "b"]
    for e in out.entries:
        c.reserve(e.request.request_id, e.num_tokens); c.commit(e.request.request_id, e.num_tokens)
    s.update(out, {})
    peak = 0
    for _ in range(200):
        if not s.has_unfinished():
            break
        out = s.schedule()
        for e in out.entries:
            c.reserve(e.request.request_id, e.num_tokens)   # never OutOfPages
            c.commit(e.request.request_id, e.num_tokens)
        peak = max(peak, 9 - c.groups[1].pool.num_free)
        s.update(out, {e.request.request_id: 7 for e in out.entries if e.samples})
        c.check()
    assert not s.has_unfinished() and s.num_preemptions == 0 and all(r.finish_reason == FinishReason.LENGTH for r in reqs)
    assert peak <= 8 and c.groups[0].pool.num_free == 16 and c.groups[1].pool.num_free == 9


def test_optimistic_admission_preempts_the_newest_when_pages_run_out():
    c = _cache(num_pages=6, page_size=4)
    s = Scheduler(c, max_num_seqs=4, max_num_batched_tokens=64, policy="optimistic", max_positions=1000)
    a, b = _req("a", 7, max_tokens=12), _req("b", 7, max_tokens=12)
    s.add_request(a)
    s.add_request(b)
    steps = _run(s)
    assert s.num_preemptions >= 1 and b.num_preemptions >= 1 and a.num_preemptions == 0
    assert a.output_token_ids == [7] * 12 and b.output_token_ids == [7] * 12
    assert c.free_pages() == 6
    # after the preemption b is recomputed from its prompt and what it had generated
    k = next(i for i, o in enumerate(steps) if o.preempted)
    later = [e for o in steps[k + 1:] for e in o.entries if e.request is b]
    assert later[0].start == 0 and later[0].num_tokens > 7
    # a request that cannot move with the whole pool to itself fails instead of spinning
    c2 = _cache(num_pages=2, page_size=4)
    s2 = Scheduler(c2, 4, 64, policy="optimistic", max_positions=1000)
    r = _req("r", 6, max_tokens=50)
    s2.add_request(r)
    for _ in range(20):
        if not s2.has_unfinished():
            break
        out = s2.schedule()
        for e in out.entries:
            c2.reserve("r", e.num_tokens); c2.commit("r", e.num_tokens)
        s2.update(out, {"r": 7} if any(e.samples for e in out.entries) else {})
    assert r.status == RequestStatus.FAILED and "no_capacity" in r.error and c2.free_pages() == 2


@pytest.mark.parametrize("sharing", [False, True])
@pytest.mark.parametrize("seed", range(4))
def test_every_admitted_request_finishes_under_random_load(seed, sharing):
    rng = random.Random(seed)
    c = _shared_cache(num_pages=14, page_size=4) if sharing else _cache(num_pages=14, page_size=4)
    s = Scheduler(c, max_num_seqs=3, max_num_batched_tokens=rng.choice([5, 9, 32]), chunk_size=rng.choice([3, 8, 64]),
                  policy=rng.choice(["optimistic", "reserve_full"]), max_positions=1000)
    reqs = [_req(f"r{i}", rng.randint(1, 25), max_tokens=rng.randint(1, 12)) for i in range(12)]
    pending = list(reqs)
    short_plans = 0
    for _ in range(2000):
        while pending and rng.random() < 0.5:
            s.add_request(pending.pop(0))
        if not s.has_unfinished():
            if not pending:
                break
            continue
        steady = s._steady_decode()
        if steady is not None:   # the short way for steps of decoded tokens alone plans what the full procedure plans
            full = s._schedule_in_full()
            key = lambda o: [(e.request.request_id, e.start, e.num_tokens, e.samples) for e in o.entries]
            assert key(steady) == key(full) and not full.preempted and s.log[-1] == s.log[-2]
            short_plans += 1
        out = s.schedule()
        assert len({e.request.request_id for e in out.entries}) == len(out.entries) <= 3
        assert out.num_tokens <= s.max_num_batched_tokens
        for e in out.entries:
            assert e.start == c.length(e.request.request_id)
            c.reserve(e.request.request_id, e.num_tokens)
            c.commit(e.request.request_id, e.num_tokens, e.request.token_slice(e.start, e.num_tokens))
        s.update(out, {e.request.request_id: 7 for e in out.entries if e.samples})
        c.check()
    assert short_plans > 0
    assert all(r.is_finished() for r in reqs)
    ok = [r for r in reqs if r.status == RequestStatus.FINISHED]
    assert all(r.get_num_generated_tokens() == r.sampling_params.max_tokens for r in ok)
    assert all("no_capacity" in r.error for r in reqs if r.status == RequestStatus.FAILED)
    assert c.free_pages() == 14 and not c.requests


def test_a_later_request_begins_after_the_pages_it_shares():
    c = _shared_cache(num_pages=8, page_size=4)
    s = Scheduler(c, max_num_seqs=4, max_num_batched_tokens=64, max_positions=1000)
    a = _req("a", 14, max_tokens=3)
    s.add_request(a)
    _run(s)
    assert a.num_cached_tokens == 0 and c.groups[0].pool.num_idle == 4      # 14 + 3 - 1 computed tokens: 4 whole pages
    b, d = _req("b", 14, max_tokens=2), _req("d", 9, max_tokens=2)        # the same beginnings (1, 2, 3, ...)
    s.add_request(b)
    s.add_request(d)
    out = s.schedule()
    shape = [(e.request.request_id, e.start, e.num_tokens, e.samples) for e in out.entries]
    assert shape == [("b", 12, 2, True), ("d", 8, 1, True)]                  # never the page of the last token
    assert b.num_cached_tokens == 12 and d.num_cached_tokens == 8
    assert c.table("b", 0)[:2] == c.table("d", 0)[:2] and c.groups[0].pool.refs(c.table("b", 0)[0]) == 2
    for e in out.entries:
        c.reserve(e.request.request_id, e.num_tokens)
        c.commit(e.request.request_id, e.num_tokens, e.request.token_slice(e.start, e.num_tokens))
    s.update(out, {"b": 7, "d": 7})
    _run(s)
    c.check()
    assert c.free_pages() == 8 and c.stats()["prefix_hit_tokens"] == 20
    # shared pages are not counted twice: with 8 pages, two requests of 7 pages' length run together
    # when six of the pages are the same
    c2 = _shared_cache(num_pages=8, page_size=4)
    s2 = Scheduler(c2, max_num_seqs=4, max_num_batched_tokens=64, max_positions=1000)
    first = _req("p", 25, max_tokens=20)
    s2.add_request(first)
    out = s2.schedule()
    c2.reserve("p", 25)
    c2.commit("p", 25, first.token_slice(0, 25))
    s2.update(out, {"p": 7})
    second = _req("q", 25, max_tokens=2)
    s2.add_request(second)
    out = s2.schedule()
    assert [(e.request.request_id, e.start, e.num_tokens) for e in out.entries] == [("p", 25, 1), ("q", 24, 1)]
    assert c2.free_pages() == 1 and not out.preempted


def test_token_slice_equals_a_slice_of_all_tokens():
    r = _req("a", 4, max_tokens=9)
    r.output_token_ids = [5, 6, 7]
    joined = r.all_token_ids()
    for s in range(7):
        for n in range(1, 8 - s):
            assert r.token_slice(s, n) == joined[s:s + n]
