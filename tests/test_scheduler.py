"""The scheduler's decisions, without a device: a stand-in 'model' derives the next
token from the tokens so far, so that generations can be compared between a huge
cache and one so small that requests are preempted and recomputed."""

import pytest

from cwm_amd.cache import CacheManager
from cwm_amd.engine.scheduler import FINISHED, Request, Scheduler
from cwm_amd.parts import PagedKVSpec

VOCAB = 97


def next_token(tokens):
    acc = 7
    for t in tokens:
        acc = (acc * 31 + t + 1) % 1000003
    return acc % VOCAB


def run(prompts, num_pages, page_size=4, max_batch=4, budget=16, max_gen=12, stop=(), window=None, trace=None, headroom=0):
    specs = [PagedKVSpec(1, 8, None), PagedKVSpec(1, 8, window)]
    manager = CacheManager(specs, page_size, num_pages, max_batch)
    sched = Scheduler(manager, max_batch, budget, headroom=headroom)
    for i, p in enumerate(prompts):
        sched.add(Request(rid=i, prompt=list(p), max_len=len(p) + max_gen))
    steps = 0
    while sched.has_work():
        batch = sched.schedule()
        total = sum(item.count for item in batch)
        assert total <= budget, "token budget exceeded"
        assert len({item.request.rid for item in batch}) == len(batch)
        assert len(sched.running) <= max_batch
        toks = []
        for item, portion in zip(batch, sched.portions(batch)):
            assert portion.tokens == item.request.all_tokens()[item.start : item.start + item.count]
            assert item.start == manager.length(item.request.rid) == item.request.cached
            manager.advance(item.request.rid, item.count)
            if item.wants_logits:
                assert item.start + item.count == len(item.request)
                toks.append(next_token(item.request.all_tokens()))
        if trace is not None:
            trace.append([(item.request.rid, item.count) for item in batch])
        sched.step_done(batch, toks, set(stop))
        manager.check()
        steps += 1
        assert steps < 5000, "the scheduler does not finish"
    assert manager.live_requests() == []
    assert manager.free_pages() == [g.pool.num_pages for g in manager.groups]
    return {r.rid: r for r in sched.finished}, sched


PROMPTS = [[1, 2, 3, 4, 5, 6, 7, 8, 9], [5] * 30, [9, 8, 7], [2, 4, 6, 8, 10, 12], [11] * 17, [3, 1, 4, 1, 5, 9, 2, 6]]


def expected(prompt, max_gen, stop=()):
    toks = list(prompt)
    out = []
    for _ in range(max_gen):
        t = next_token(toks)
        toks.append(t)
        out.append(t)
        if t in stop:
            break
    return out


def test_every_request_finishes_with_the_right_tokens():
    done, sched = run(PROMPTS, num_pages=1000)
    assert sorted(done) == list(range(len(PROMPTS)))
    for i, p in enumerate(PROMPTS):
        assert done[i].generated == expected(p, 12)
        assert done[i].finish_reason == "length" and done[i].preemptions == 0


def test_tiny_pool_preempts_and_recomputes_to_the_same_tokens():
    trace = []
    done, sched = run(PROMPTS, num_pages=14, trace=trace)
    assert any(e.startswith("preempt") for e in sched.events), "the pool was meant to be too small"
    for i, p in enumerate(PROMPTS):
        assert done[i].generated == expected(p, 12), f"request {i} after {done[i].preemptions} preemptions"


def test_preemption_takes_the_shortest_running_request():
    done, sched = run([[1] * 20, [2] * 6], num_pages=9, max_gen=12, budget=64)
    first = next(e for e in sched.events if e.startswith("preempt"))
    assert first == "preempt 1"
    assert done[0].preemptions == 0 and done[1].preemptions >= 1


def test_parked_requests_come_back_before_new_ones():
    done, sched = run([[1] * 20, [2] * 6, [3] * 5], num_pages=9, max_batch=2, max_gen=12, budget=64)
    events = sched.events
    parked_back = [i for i, e in enumerate(events) if e == "admit 1"]
    assert len(parked_back) >= 2
    assert events.index("admit 2") > parked_back[1]


def test_decode_tokens_come_first_and_prompts_are_cut_to_the_budget():
    trace = []
    run([[1] * 40, [2] * 3, [3] * 50], num_pages=1000, budget=16, max_gen=4, trace=trace)
    assert trace[0] == [(0, 16)]
    assert trace[1] == [(0, 16)]
    assert trace[2] == [(0, 8), (1, 3), (2, 5)]  # the rest of 0, all of 1, the start of 2 share a step
    assert trace[3][:2] == [(0, 1), (1, 1)] and trace[3][2] == (2, 14)  # decoded tokens first, then the portion
    assert all(sum(c for _, c in step) <= 16 for step in trace)


def test_stop_token_ends_a_request_and_is_kept():
    p = PROMPTS[0]
    full = expected(p, 12)
    stop = full[4]
    done, _ = run([p], num_pages=100, stop=[stop])
    cut = full.index(stop)
    assert done[0].generated == full[: cut + 1] and done[0].finish_reason == "stop"


def test_a_request_too_long_for_the_cache_ends_with_reason_cache():
    done, sched = run([[1] * 50, [2] * 5], num_pages=4, page_size=4, max_gen=3)
    assert done[0].finish_reason == "cache" and done[0].generated == []
    assert done[1].generated == expected([2] * 5, 3)


def test_a_lone_request_that_outgrows_the_cache_stops():
    done, _ = run([[1] * 6], num_pages=3, page_size=4, max_gen=50)
    assert done[0].finish_reason == "cache"
    assert done[0].generated == expected([1] * 6, 50)[: len(done[0].generated)]
    assert 6 + len(done[0].generated) - 1 <= 12


def test_window_group_lets_longer_sequences_fit():
    # 8 pages of 4 tokens hold 32 tokens; the windowed group frees pages as it goes, the keep-all group is the limit
    done, _ = run([[1] * 10], num_pages=8, page_size=4, max_gen=20, window=6)
    assert done[0].finish_reason == "length" and len(done[0].generated) == 20


def test_no_admission_and_preemption_in_turns_under_page_pressure():
    """Two requests that cannot both grow to their full length in the pool: the second is let in
    only when its known tokens fit beside the first, is preempted at most once when both outgrow
    the pool, and then waits until it fits again, instead of being admitted with a part of its
    prompt, losing it as the shortest request, and coming back every other step."""
    prompts = [[1] * 18, [2] * 18]
    trace = []
    done, sched = run(prompts, num_pages=10, page_size=4, max_batch=4, budget=16, max_gen=22, trace=trace)
    for i, p in enumerate(prompts):
        assert done[i].generated == expected(p, 22)
    assert sched.n_preemptions <= 1
    scheduled = sum(c for step in trace for _, c in step)
    needed = sum(len(p) + 22 - 1 for p in prompts)  # every token but the last generated one runs once
    assert scheduled <= needed + 18 + 22  # at most one request is computed twice
    # with room to decode asked for at admission there is no preemption at all: the second waits
    done, sched = run(prompts, num_pages=10, page_size=4, max_batch=4, budget=16, max_gen=22, headroom=22)
    assert sched.n_preemptions == 0
    for i, p in enumerate(prompts):
        assert done[i].generated == expected(p, 22)


def test_a_request_joins_others_only_when_it_fits_whole():
    sched_trace = []
    # 12 pages of 4: the first request holds 10 after its prompt; the second's 12 tokens need 3
    done, sched = run([[1] * 40, [2] * 12], num_pages=12, page_size=4, budget=64, max_gen=4, trace=sched_trace)
    events = list(sched.events)
    assert events.index("admit 1") > events.index("finish 0 length")
    assert sched.n_preemptions == 0
    # a shorter first request leaves room for it at once
    done, sched = run([[1] * 30, [2] * 12], num_pages=12, page_size=4, budget=64, max_gen=4)
    events = list(sched.events)
    assert events.index("admit 1") < events.index("finish 0 length")


def test_events_and_finished_requests_do_not_pile_up():
    manager = CacheManager([PagedKVSpec(1, 8, None)], 4, 64, 2)
    sched = Scheduler(manager, 2, 8)
    assert sched.events.maxlen is not None
    seen = []
    sched.on_event = lambda kind, request: seen.append((kind, request.rid))
    sched.add(Request(rid="x", prompt=[1, 2, 3], max_len=4))
    batch = sched.schedule()
    for item in batch:
        manager.advance(item.request.rid, item.count)
    sched.step_done(batch, [5], set())
    assert seen == [("admit", "x"), ("finish", "x")]
    assert [r.rid for r in sched.finished] == ["x"]


def test_empty_prompt_is_refused():
    manager = CacheManager([PagedKVSpec(1, 8, None)], 4, 8, 2)
    with pytest.raises(ValueError):
        Scheduler(manager, 2, 8).add(Request(rid=0, prompt=[], max_len=4))


@pytest.mark.parametrize("seed", range(60))
def test_random_workloads_give_the_tokens_of_an_undisturbed_run(seed):
    """Random prompts, arrival times, pools, page sizes, windows, budgets, headroom and decode
    bursts: whatever is preempted, recomputed or cut, a request's tokens are those it would
    get alone, and the books balance after every step."""
    import random

    rng = random.Random(seed)
    page_size = rng.choice([1, 2, 4, 8, 16])
    max_batch = rng.choice([1, 2, 4, 6])
    budget = rng.choice([2, 5, 16, 64])
    window = rng.choice([None, 3, 8, 20])
    headroom = rng.choice([0, 0, 4, 128])
    burst = rng.choice([1, 1, 3, 10])
    stop = {rng.randrange(VOCAB)} if rng.random() < 0.5 else set()
    n_requests = rng.randrange(1, 12)
    todo = []
    for i in range(n_requests):
        prompt = [rng.randrange(VOCAB) for _ in range(rng.choice([1, 2, 7, 19, 40, 90]))]
        todo.append((rng.randrange(0, 30), Request(rid=i, prompt=prompt, max_len=len(prompt) + rng.choice([1, 2, 9, 33, 80]))))
    longest = max(r.max_len for _, r in todo)
    # from a pool that preempts all the time to one that never does; always enough for the longest request alone
    pages_alone = -(-longest // page_size) + 1
    num_pages = pages_alone + rng.choice([0, 1, 3, 5, 12, 40, 400])
    specs = [PagedKVSpec(1, 8, None), PagedKVSpec(1, 8, window)]
    manager = CacheManager(specs, page_size, num_pages, max_batch)
    sched = Scheduler(manager, max_batch, budget, headroom=headroom)
    todo.sort(key=lambda pair: pair[0])
    steps = 0
    while todo or sched.has_work():
        while todo and todo[0][0] <= steps:
            sched.add(todo.pop(0)[1])
        steps += 1
        assert steps < 20000, "the scheduler does not finish"
        if not sched.has_work():
            continue
        batch = sched.schedule()
        assert sum(item.count for item in batch) <= budget
        assert len(sched.running) <= max_batch
        decode_only = bool(batch) and all(item.count == 1 and item.wants_logits and item.request.generated for item in batch)
        n = sched.reserve_burst(batch, burst) if decode_only and burst > 1 else 1
        if n > 1:
            rows = []
            sofar = [item.request.all_tokens() for item in batch]
            for _ in range(n):
                for item in batch:
                    manager.advance(item.request.rid, 1)
                row = [next_token(toks) for toks in sofar]
                for toks, t in zip(sofar, row):
                    toks.append(t)
                rows.append(row)
            sched.burst_done(batch, rows, stop)
        else:
            toks = []
            for item, portion in zip(batch, sched.portions(batch)):
                assert portion.tokens == item.request.all_tokens()[item.start : item.start + item.count]
                assert item.start == manager.length(item.request.rid) == item.request.cached
                manager.advance(item.request.rid, item.count)
                if item.wants_logits:
                    toks.append(next_token(item.request.all_tokens()))
            sched.step_done(batch, toks, stop)
        manager.check()
    assert manager.live_requests() == []
    assert manager.free_pages() == [g.pool.num_pages for g in manager.groups]
    done = {r.rid: r for r in sched.finished}
    assert sorted(done) == list(range(n_requests))
    for r in done.values():
        want = expected(r.prompt, r.max_len - len(r.prompt), stop)
        assert r.generated == want, (r.rid, r.finish_reason)
        assert r.finish_reason == ("stop" if want[-1] in stop else "length")
