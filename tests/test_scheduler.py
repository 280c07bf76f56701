"""The scheduler's decisions, on the cache manager's bookkeeping alone (no GPU, no model)."""
import pytest

from simply_amd.cache import CacheManager
from simply_amd.engine.scheduler import Request, Scheduler, Status
from simply_amd.parts.base import PagedKVNeed
from simply_amd.sampling import SamplingParams


def make(num_pages=32, page_size=4, slots=4, budget=16, max_len=128, window=8):
    needs = [(PagedKVNeed(1, 16, window), None), (PagedKVNeed(1, 16, None), None)]
    cache = CacheManager(needs, page_size=page_size, num_pages=num_pages, num_slots=slots, max_seq_len=max_len)
    return cache, Scheduler(cache, max_num_issue_tokens=budget, max_seq_len=max_len)


def req(rid, n, steps=4, **kw):
    return Request(rid, list(range(1, n + 1)), SamplingParams(temperature=0.0, max_decode_steps=steps, **kw))


def run_step(sched, out, token=7):
    toks = [token if s.samples else None for s in out.scheduled]
    lps = [0.0 if s.samples else None for s in out.scheduled]
    return sched.update(out.scheduled, toks, lps)


def test_budget_cuts_one_prompt_and_decodes_go_first():
    """After simply/utils/ragged_paged_attention_test.py:758-795 (issue_lens): requests get all they want
    in order until the budget runs out; one gets a partial portion, the rest nothing."""
    cache, sched = make(budget=16)
    for rid, n in (("a", 5), ("b", 20), ("c", 3)):
        sched.add(req(rid, n))
    out = sched.schedule()
    assert [(s.request.request_id, s.start, s.num_tokens, s.samples) for s in out.scheduled] == \
        [("a", 0, 5, True), ("b", 0, 11, False)]
    run_step(sched, out)
    out = sched.schedule()
    # a decodes (1 token) first, then b's remaining 9, then c is admitted with its 3
    assert [(s.request.request_id, s.start, s.num_tokens, s.samples) for s in out.scheduled] == \
        [("a", 5, 1, True), ("b", 11, 9, True), ("c", 0, 3, True)]
    run_step(sched, out)
    out = sched.schedule()
    assert [(s.request.request_id, s.num_tokens) for s in out.scheduled] == [("a", 1), ("b", 1), ("c", 1)]
    cache.check()


def test_finish_reasons_and_release():
    cache, sched = make()
    sched.add(Request("e", [1, 2, 3], SamplingParams(temperature=0.0, max_decode_steps=10), eos_ids=(9,)))
    sched.add(Request("l", [1, 2, 3], SamplingParams(temperature=0.0, max_decode_steps=2), eos_ids=(5,)))
    sched.add(Request("i", [1, 2, 3], SamplingParams(temperature=0.0, max_decode_steps=3, ignore_eos=True), eos_ids=(9,)))
    sched.add(Request("m", [1, 2, 3], SamplingParams(temperature=0.0, max_decode_steps=10, max_seq_len=5)))
    done = {}
    for _ in range(5):
        out = sched.schedule()
        for r in run_step(sched, out, token=9):
            done[r.request_id] = (r.finish_reason, len(r.output_token_ids), r.is_truncated)
    assert done == {"e": ("eos", 1, False), "l": ("length", 2, True), "i": ("length", 3, True),
                    "m": ("max_seq_len", 2, True)}
    assert not sched.has_work()
    assert all(g.pool.num_free == 32 for g in cache.groups) and cache.slots.num_free == 4
    cache.check()


def test_no_slot_waits():
    cache, sched = make(slots=2, budget=64)
    for rid in "abc":
        sched.add(req(rid, 4, steps=2))
    out = sched.schedule()
    assert [s.request.request_id for s in out.scheduled] == ["a", "b"]
    run_step(sched, out)
    out = sched.schedule()
    assert [s.request.request_id for s in out.scheduled] == ["a", "b"]
    assert [r.request_id for r in run_step(sched, out)] == ["a", "b"]
    out = sched.schedule()
    assert [s.request.request_id for s in out.scheduled] == ["c"]


def test_admission_needs_room_for_the_whole_prompt():
    cache, sched = make(num_pages=6, page_size=4, budget=64, window=None)
    sched.add(req("a", 14, steps=8))     # 4 pages
    sched.add(req("b", 20, steps=2))     # would need 5, only 2 are free: it waits
    sched.add(req("c", 3, steps=2))      # would fit, but requests are admitted in order of arrival
    out = sched.schedule()
    assert [(s.request.request_id, s.num_tokens, s.samples) for s in out.scheduled] == [("a", 14, True)]
    assert [r.request_id for r in sched.waiting] == ["b", "c"]
    cache.check()


def test_later_prompt_portion_shrinks_to_free_pages():
    cache, sched = make(num_pages=8, page_size=4, budget=10, window=None)
    sched.add(req("a", 3, steps=30))
    sched.add(req("b", 26, steps=2))     # 7 pages: admitted (all 8 are free but one), runs in portions of the budget
    out = sched.schedule()
    assert [(s.request.request_id, s.num_tokens) for s in out.scheduled] == [("a", 3), ("b", 7)]
    run_step(sched, out)
    # a grows meanwhile and takes the pages that b's last portion would have needed
    for want_b in (9, 8):
        out = sched.schedule()
        assert [(s.request.request_id, s.num_tokens) for s in out.scheduled] == [("a", 1), ("b", want_b)]
        run_step(sched, out)
        cache.groups[0].pool.take(0)
    a_pages = len(cache.groups[0].pages_of("a"))
    assert a_pages == 2
    cache.check()


def test_out_of_pages_preempts_the_newest_and_recomputes():
    cache, sched = make(num_pages=4, page_size=4, budget=64, window=None)
    a, b = req("a", 7, steps=20), req("b", 7, steps=20)
    sched.add(a)
    sched.add(b)
    out = sched.schedule()
    assert [s.num_tokens for s in out.scheduled] == [7, 7]      # 2 pages each: the pool is full
    run_step(sched, out)
    out = sched.schedule()                                       # position 7 still fits in the second page
    assert [s.num_tokens for s in out.scheduled] == [1, 1] and not out.preempted
    run_step(sched, out)
    out = sched.schedule()                                       # position 8 needs a third page: b gives way
    assert [r.request_id for r in out.preempted] == ["b"]
    assert [(s.request.request_id, s.start, s.num_tokens) for s in out.scheduled] == [("a", 8, 1)]
    assert b.status is Status.WAITING and b.num_computed == 0 and len(b.output_token_ids) == 2
    assert sched.waiting[0] is b
    cache.check()
    run_step(sched, out)
    # a runs on; b comes back only when pages are free again, with prompt and generated tokens as one portion
    for _ in range(3):
        out = sched.schedule()
        assert [s.request.request_id for s in out.scheduled] == ["a"]
        run_step(sched, out)
    while a.status is not Status.FINISHED:
        out = sched.schedule()
        run_step(sched, out)
    out = sched.schedule()
    assert [(s.request.request_id, s.start, s.num_tokens, s.samples) for s in out.scheduled] == [("b", 0, 9, True)]
    assert b.num_preemptions == 1
    cache.check()


def test_request_that_fits_nowhere_ends_truncated():
    cache, sched = make(num_pages=2, page_size=4, budget=64, max_len=128, window=None)
    with pytest.raises(ValueError):
        sched.add(req("big", 8))       # 8 tokens fill the 2 pages: nothing could be generated
    r = req("r", 5, steps=50)
    sched.add(r)
    done = []
    for _ in range(10):
        if not sched.has_work():
            break
        out = sched.schedule()
        done += out.finished + run_step(sched, out)
    assert done == [r] and r.finish_reason == "max_seq_len" and r.num_tokens == 8
    assert all(g.pool.num_free == 2 for g in cache.groups)


def test_empty_prompt_and_bad_params_are_refused():
    _, sched = make()
    with pytest.raises(ValueError):
        sched.add(Request("x", [], SamplingParams()))
    with pytest.raises(ValueError):
        sched.add(Request("y", [1], SamplingParams(top_p=0.0)))
    with pytest.raises(ValueError):
        sched.add(Request("z", [1], SamplingParams(temperature=-1.0)))


def test_max_input_len_keeps_the_tail():
    _, sched = make()
    r = Request("t", list(range(30)), SamplingParams(max_input_len=10))
    sched.add(r)
    assert r.prompt_token_ids == list(range(20, 30))


def test_decoding_requests_ask_the_cache_once():
    """A step of decoding requests that all fit costs a fixed number of passes over the live requests, not one
    per request; the decisions are those of the one-by-one path (oldest first, one token each)."""
    cache, sched = make(num_pages=256, slots=32, budget=64, max_len=128)
    for i in range(32):
        sched.add(req(f"r{i}", 2, steps=50))
    run_step(sched, sched.schedule())
    run_step(sched, sched.schedule())
    calls = []
    original = cache.can_reserve
    cache.can_reserve = lambda wants: calls.append(len(wants)) or original(wants)
    out = sched.schedule()
    assert [(s.request.request_id, s.num_tokens, s.samples) for s in out.scheduled] == \
        [(f"r{i}", 1, True) for i in range(32)]
    assert len(calls) <= 3 and max(calls) == 32
    cache.check()


@pytest.mark.parametrize("seed", range(12))
@pytest.mark.parametrize("window,page_size,slots,budget,ahead", [(8, 4, 4, 16, 8), (50, 16, 6, 64, 16)])
def test_a_windowed_pool_as_tight_as_the_engine_makes_it(seed, window, page_size, slots, budget, ahead):
    """The engine gives a windowed group only the pages that its requests can hold at once
    (`CacheManager(max_step_tokens=...)`), not as many as the group that keeps everything.  Random long prompts and
    runs of decode steps that reserve ahead and end early, as `LMInterface.step` and `Executor.decode_many` do them
    (pages for the whole run reserved first, `mark_issued` for the steps that ran): admission, portions that shrink
    to the free pages, requests left out of a step and preemption never run the tight pool dry, lose a page or
    finish a request for want of room."""
    import numpy as np

    from simply_amd.cache import OutOfPages

    rng = np.random.default_rng(1000 * window + seed)
    max_len = 40 * page_size
    needs = [(PagedKVNeed(1, 16, window), None), (PagedKVNeed(1, 16, None), None)]
    pages = slots * (max_len // page_size)
    cache = CacheManager(needs, page_size=page_size, num_pages=pages, num_slots=slots, max_seq_len=max_len,
                         max_step_tokens=max(budget, slots * ahead))
    windowed = next(g for g in cache.groups if g.window is not None)
    assert windowed.pool.num_pages < pages // 2
    sched = Scheduler(cache, max_num_issue_tokens=budget, max_seq_len=max_len)
    todo = [req(f"r{i}", int(rng.integers(1, max_len - 40)), steps=int(rng.integers(1, 40)), ignore_eos=True)
            for i in range(14)]
    finished, arrivals = [], 0
    for _ in range(4000):
        while todo and rng.random() < 0.3:
            sched.add(todo.pop())
        if not sched.has_work():
            if not todo:
                break
            sched.add(todo.pop())
        out = sched.schedule()
        finished += out.finished
        if not out.scheduled:
            continue
        cache.check()
        decoding = all(s.num_tokens == 1 and s.samples for s in out.scheduled)
        n = 1
        if decoding and not sched.waiting and len(out.scheduled) == len(sched.running):
            n = ahead
            for s in out.scheduled:
                n = min(n, s.request.params.max_decode_steps - len(s.request.output_token_ids))
            while n > 1 and not cache.can_reserve([(s.request.request_id, s.start, n) for s in out.scheduled]):
                n //= 2
        wants = [(s.request.request_id, s.start, max(s.num_tokens, n)) for s in out.scheduled]
        cache.reserve_all(wants)       # as the step function does (OutOfPages here would fail the test)
        ran = int(rng.integers(1, n + 1)) if n > 1 else 1        # a run may end early
        live = list(out.scheduled)
        for k in range(ran):
            now = [type(s)(s.request, s.start + k, s.num_tokens, s.samples) for s in live]
            finished += sched.update(now, [7] * len(now), [0.0] * len(now)) if n > 1 else run_step(sched, out)
            live = [s for s in live if s.request.status is Status.RUNNING]
            if len(live) < len(now):
                ran = k + 1
                break
        cache.mark_issued([(s.request.request_id, s.start, s.num_tokens if n == 1 else ran) for s in out.scheduled
                           if s.request.request_id in cache.requests])
        cache.check()
    assert not sched.has_work() and not todo
    assert len(finished) == 14 and all(r.finish_reason in ("length", "max_seq_len") for r in finished), \
        [(r.request_id, r.finish_reason) for r in finished]
    assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups) and cache.slots.num_free == slots
