"""The scheduler's decisions, on the host alone."""
import pytest
import torch

from transformers_neuronx_amd.cache import CacheManager, OutOfPages
from transformers_neuronx_amd.engine.scheduler import Request, Scheduler
from transformers_neuronx_amd.parts.base import CacheNeed
from transformers_neuronx_amd.sampling import SamplingParams


def _sched(num_pages=16, page=16, max_seqs=4, budget=64, max_len=256, portion=None):
    cache = CacheManager({0: CacheNeed("paged", kv_heads=1, head_size=16)}, page, num_pages, max_seqs,
                         torch.float32, "cpu", allocate=False)
    return Scheduler(cache, max_seqs, budget, max_len, portion), cache


def _req(rid, n, new=4, **kw):
    return Request(rid, list(range(3, 3 + n)), SamplingParams(max_new_tokens=new, do_sample=False, **kw))


def _step(s, cache, token=7):
    runs = s.schedule()
    for r in runs:
        cache.advance(r.request.req_id, r.count)
    ended = s.update(runs, [token if r.samples else None for r in runs])
    cache.check()
    return runs, ended


def test_budget_cuts_prompts_into_portions():
    s, cache = _sched(budget=64)
    s.add(_req("a", 100))
    s.add(_req("b", 30))
    runs, _ = _step(s, cache)
    assert [(r.request.req_id, r.start, r.count, r.samples) for r in runs] == [("a", 0, 64, False)]
    runs, _ = _step(s, cache)
    assert [(r.request.req_id, r.start, r.count, r.samples) for r in runs] == [("a", 64, 36, True), ("b", 0, 28, False)]
    runs, _ = _step(s, cache)          # a decodes first, then b's prompt goes on
    assert [(r.request.req_id, r.start, r.count) for r in runs] == [("a", 100, 1), ("b", 28, 2)]
    assert runs[0].samples and runs[1].samples


def test_portion_limit_and_decode_first():
    s, cache = _sched(budget=40, portion=16)
    s.add(_req("a", 20, new=10))
    for expect in ([("a", 0, 16)], [("a", 16, 4)]):
        runs, _ = _step(s, cache)
        assert [(r.request.req_id, r.start, r.count) for r in runs] == expect
    s.add(_req("b", 50))
    runs, _ = _step(s, cache)
    assert [(r.request.req_id, r.start, r.count) for r in runs] == [("a", 20, 1), ("b", 0, 16)]


def test_finishing_frees_everything():
    s, cache = _sched()
    s.add(_req("a", 5, new=3))
    s.add(_req("b", 5, new=8, eos_token_id=7))
    s.add(_req("c", 5, new=8, eos_token_id=7, ignore_eos=True))
    _, ended = _step(s, cache, token=7)           # prompts; b ends at once on eos
    assert [r.req_id for r in ended] == ["b"] and ended[0].finish_reason == "eos"
    _, ended = _step(s, cache, token=7)
    assert ended == []
    _, ended = _step(s, cache, token=7)
    assert [r.req_id for r in ended] == ["a"] and ended[0].finish_reason == "length" and ended[0].output == [7, 7, 7]
    while s.has_work:
        _step(s, cache, token=7)
    assert cache.groups["full"].pool.num_free == 16 and cache.slots.num_free == 4 and not cache.requests
    assert [r.req_id for r in s.finished] == ["b", "a", "c"]


def test_length_limits():
    s, _ = _sched(max_len=32)
    with pytest.raises(ValueError, match="positions"):
        s.add(_req("a", 30, new=4))
    s.add(_req("b", 30, new=3))                   # 30 + 3 - 1 positions: fits
    with pytest.raises(ValueError, match="empty"):
        s.add(Request("c", [], SamplingParams()))


def test_slots_bound_admission():
    s, cache = _sched(max_seqs=2, budget=512)
    for i in range(3):
        s.add(_req(f"r{i}", 4, new=2))
    runs, _ = _step(s, cache)
    assert [r.request.req_id for r in runs] == ["r0", "r1"]
    runs, ended = _step(s, cache)
    assert {r.req_id for r in ended} == {"r0", "r1"}
    runs, _ = _step(s, cache)
    assert [r.request.req_id for r in runs] == ["r2"]


def test_pages_run_out_newest_goes_back_and_is_computed_again():
    s, cache = _sched(num_pages=4, page=16, budget=512)      # 64 tokens of cache in all
    s.add(_req("a", 30, new=20))
    s.add(_req("b", 30, new=20))
    _step(s, cache)
    assert [r.req_id for r in s.running] == ["a", "b"] and cache.groups["full"].pool.num_free == 0
    preempted_at = None
    for i in range(60):
        if not s.has_work:
            break
        runs, _ = _step(s, cache)
        if s.num_preemptions and preempted_at is None:
            preempted_at = i
            assert [r.req_id for r in s.running] == ["a"]            # the newest one gave way
            assert s.waiting[0].req_id == "b" and s.waiting[0].num_computed == 0
            kept = list(s.waiting[0].output)
            assert kept                                               # what it generated is kept
            assert not cache.has("b")
    assert preempted_at is not None and not s.has_work
    a, b = s.finished if s.finished[0].req_id == "a" else s.finished[::-1]
    assert len(a.output) == 20 and len(b.output) == 20 and b.preemptions >= 1 and a.preemptions == 0
    assert cache.groups["full"].pool.num_free == 4


def test_nothing_is_admitted_while_pages_are_short():
    s, cache = _sched(num_pages=3, page=16, budget=512)
    s.add(_req("a", 40, new=30))
    _step(s, cache)
    s.add(_req("b", 20, new=2))                   # needs 2 pages; none free
    runs, _ = _step(s, cache)
    assert [r.request.req_id for r in runs] == ["a"] and [r.req_id for r in s.waiting] == ["b"]


def test_a_lone_request_that_cannot_fit_raises():
    s, cache = _sched(num_pages=2, page=16, budget=512)
    s.add(_req("a", 40, new=2))
    with pytest.raises(OutOfPages, match="alone"):
        s.schedule()
    s2, cache2 = _sched(num_pages=2, page=16, budget=512)
    s2.add(_req("a", 30, new=20))
    _step(s2, cache2)
    with pytest.raises(OutOfPages, match="alone"):
        for _ in range(10):
            _step(s2, cache2)


def test_decisions_depend_on_arrivals_and_lengths_only():
    def trace(tokens):
        s, cache = _sched(num_pages=6, page=16, budget=48)
        for i, n in enumerate((50, 9, 33, 20)):
            s.add(_req(f"r{i}", n, new=6))
        out = []
        it = iter(tokens)
        while s.has_work:
            runs, _ = _step(s, cache, token=next(it))
            out.append([(r.request.req_id, r.start, r.count) for r in runs])
        return out
    assert trace(iter(range(10, 1000))) == trace(iter(range(500, 1500)))


def test_prompts_first_holds_decoding_until_every_prompt_is_in():
    cache = CacheManager({0: CacheNeed("paged", kv_heads=1, head_size=16)}, 16, 32, 4, torch.float32, "cpu",
                         allocate=False)
    s = Scheduler(cache, 4, 40, 256, prompts_first=True)
    s.add(_req("a", 30, new=5))
    s.add(_req("b", 60, new=5))
    seen = []
    for _ in range(4):
        runs, _ = _step(s, cache)
        seen.append([(r.request.req_id, r.start, r.count) for r in runs])
    # a is in after the first step and waits, with one token drawn, until b's prompt is in too
    assert seen == [[("a", 0, 30), ("b", 0, 10)], [("b", 10, 40)], [("b", 50, 10)], [("a", 30, 1), ("b", 60, 1)]]


def test_a_step_recorded_before_its_tokens_are_known():
    """`record` plans on with PENDING tokens, `resolve` fills them in one step late: an end by length is
    known at once, an end-of-sequence token ends the request when it is read, and the run that the request
    had in the step started meanwhile gives it nothing."""
    from transformers_neuronx_amd.engine.scheduler import PENDING
    s, cache = _sched()
    s.add(_req("a", 5, new=3, eos_token_id=9))
    s.add(_req("b", 6, new=8, eos_token_id=9))

    def start():
        runs = s.schedule()
        for r in runs:
            cache.advance(r.request.req_id, r.count)
        s.record(runs)
        cache.check()
        return runs

    first = start()                                  # both prompts; both draw a token
    a, b = first[0].request, first[1].request
    assert a.output == [PENDING] and b.output == [PENDING] and a.decoding and b.decoding
    second = start()                                 # planned with the pending tokens: one token each
    assert [(r.request.req_id, r.start, r.count, r.out_index) for r in second] == [("a", 5, 1, 1), ("b", 6, 1, 1)]
    assert a.span(5, 1) == [PENDING]
    assert s.resolve(first, [4, 9]) == [4, 9]        # b drew its end-of-sequence token in the first step
    assert b.finished and b.finish_reason == "eos" and b.output == [9] and not cache.has("b")
    assert a.output == [4, PENDING] and not a.finished
    third = start()                                  # a alone; its third token ends it by length, at once
    assert [r.request.req_id for r in third] == ["a"] and a.finished and a.finish_reason == "length"
    assert not cache.has("a") and not s.has_work
    assert s.resolve(second, [5, 6]) == [5, None]    # b's token of the second step is dropped
    assert s.resolve(third, [9]) == [9]              # the last token happens to be the end-of-sequence one
    assert a.output == [4, 5, 9] and a.finish_reason == "eos" and b.output == [9]
    assert [r.req_id for r in s.finished] == ["b", "a"]
    cache.check()


def test_a_request_ends_when_its_time_is_up():
    """`max_time` (stopping_criteria.py:15-35): the first token that comes later than that ends the request,
    with the reason "time"; a request with time to spare is not touched."""
    import time
    from transformers_neuronx_amd.engine.scheduler import Request, Scheduler
    from transformers_neuronx_amd.sampling import SamplingParams
    cache = CacheManager({0: CacheNeed("paged")}, 16, 8, 4, torch.float32, "cpu")
    sched = Scheduler(cache, 4, 64, 128)
    slow = Request("slow", [1, 2, 3], SamplingParams(max_new_tokens=10, max_time=0.0, ignore_eos=True))
    fast = Request("fast", [4, 5], SamplingParams(max_new_tokens=3, max_time=3600.0, ignore_eos=True))
    sched.add(slow)
    sched.add(fast)
    time.sleep(0.002)
    steps = 0
    while sched.has_work:
        runs = sched.schedule()
        sched.update(runs, [7 if r.samples else None for r in runs])
        steps += 1
    assert slow.output == [7] and slow.finish_reason == "time"
    assert fast.output == [7, 7, 7] and fast.finish_reason == "length" and steps == 3
    cache.check()
    assert not cache.requests
