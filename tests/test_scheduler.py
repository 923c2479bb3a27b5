"""The scheduler's decisions, on the host, against a cache manager (no GPU): portions under the
token budget, decode before prompt, admission in order, what happens when pages run out."""
import random

import pytest

from flambeau_amd.cache import CacheManager, GroupSpec
from flambeau_amd.engine.scheduler import AdmissionError, Scheduler
from flambeau_amd.sampling import SamplingParams


def mk(n_pages=16, page=4, slots=3, max_len=64, budget=16, chunk=8, window=0, **kw):
    m = CacheManager([GroupSpec(1, 8, window)], n_pages, page, slots, max_len)
    return m, Scheduler(m, max_batch_tokens=budget, prefill_chunk_tokens=chunk, **kw)


def run_step(m, s, token=lambda r: 100 + len(r.output)):
    """What the engine does around the scheduler: reserve pages, advance, commit."""
    sched = s.schedule()
    for e in sched:
        rid = e.request.request_id
        assert e.tokens == e.request.tokens[e.request.n_computed:e.request.n_computed + len(e.tokens)]
        assert m.live[rid].n_cached == e.request.n_computed
        m.ensure(rid, e.request.n_computed + len(e.tokens))      # must never raise: the scheduler asked first
        m.advance(rid, len(e.tokens))
    done = s.commit(sched, {e.request.request_id: token(e.request) for e in sched if e.sample})
    m.check_invariants()
    return sched, done


def test_prompt_is_cut_into_portions_and_sampled_at_its_end():
    m, s = mk()
    r = s.add("a", list(range(19)), SamplingParams(max_tokens=3))
    sizes, samples = [], []
    while s.has_work():
        sched, _ = run_step(m, s)
        sizes.append([len(e.tokens) for e in sched])
        samples.append([e.sample for e in sched])
    assert sizes == [[8], [8], [3], [1], [1]]
    assert samples == [[False], [False], [True], [True], [True]]
    assert r.output == [100, 101, 102] and r.finish_reason == "length" and r.status == "finished"
    assert m.free_pages() == [16] and m.n_free_slots == 3


def test_decode_rows_come_first_and_the_budget_is_shared():
    m, s = mk(budget=10, chunk=8)
    s.add("a", [1, 2, 3], SamplingParams(max_tokens=20))
    run_step(m, s)                                   # a's prompt, first token sampled
    s.add("b", list(range(30)), SamplingParams(max_tokens=2))
    s.add("c", list(range(5)), SamplingParams(max_tokens=2))
    sched, _ = run_step(m, s)
    assert [(e.request.request_id, len(e.tokens)) for e in sched] == [("a", 1), ("b", 8), ("c", 1)]
    sched, _ = run_step(m, s)                        # several portions in one step, budget 10
    assert [(e.request.request_id, len(e.tokens)) for e in sched] == [("a", 1), ("b", 8), ("c", 1)]
    assert sum(len(e.tokens) for e in sched) <= 10


def test_admission_keeps_order_and_waits_for_slots():
    m, s = mk(slots=2)
    for rid in "abc":
        s.add(rid, [1, 2, 3, 4, 5], SamplingParams(max_tokens=2))
    sched, _ = run_step(m, s)
    assert [e.request.request_id for e in sched] == ["a", "b"] and [r.request_id for r in s.waiting] == ["c"]
    run_step(m, s)                                   # a and b finish (2 tokens each)
    sched, _ = run_step(m, s)
    assert [e.request.request_id for e in sched] == ["c"]


def test_refusals_at_add():
    m, s = mk(n_pages=4, page=4, max_len=64, max_queue_depth=2)
    with pytest.raises(AdmissionError, match="empty prompt"):
        s.add("e", [])
    with pytest.raises(AdmissionError, match="needs 5 pages"):
        s.add("big", list(range(17)), SamplingParams(max_tokens=1))      # 17 cached tokens > 4 pages of 4
    s.add("fits", list(range(16)), SamplingParams(max_tokens=1))
    s.waiting.clear()
    with pytest.raises(AdmissionError, match="maximum length"):
        s.add("long", list(range(64)))
    one = SamplingParams(max_tokens=1)
    s.add("a", [1], one)
    s.add("b", [1], one)
    with pytest.raises(AdmissionError, match="queue full"):
        s.add("c", [1], one)
    s2 = mk()[1]
    s2.add("a", [1], one)
    with pytest.raises(AdmissionError, match="already known"):
        s2.add("a", [2], one)


def test_when_pages_run_out_the_newest_request_is_preempted_and_resumes():
    """Two requests of 8 + 12 tokens each need 5 pages each; the pool has 7.  The older one must
    finish without interruption; the newer is pre-empted, waits, then recomputes all it had."""
    m, s = mk(n_pages=7, page=4, slots=2, budget=16, chunk=16)
    a = s.add("a", list(range(8)), SamplingParams(max_tokens=12))
    b = s.add("b", list(range(50, 58)), SamplingParams(max_tokens=12))
    order = []
    for _ in range(200):
        if not s.has_work():
            break
        sched, done = run_step(m, s)
        order += [r.request_id for r in done]
        assert all(p.n_free >= 0 for p in m.pools)
    assert not s.has_work()
    assert order == ["a", "b"] and a.n_preempted == 0 and b.n_preempted >= 1 and s.n_preemptions >= 1
    assert len(a.output) == 12 and len(b.output) == 12
    assert b.output == [100 + i for i in range(12)]          # nothing lost or doubled across the pre-emption
    assert m.free_pages() == [7] and m.n_free_slots == 2


def test_a_preempted_request_recomputes_prompt_and_output():
    m, s = mk(n_pages=5, page=4, slots=2, budget=32, chunk=32)
    reqs = [s.add("a", list(range(6)), SamplingParams(max_tokens=10)),
            s.add("b", list(range(6)), SamplingParams(max_tokens=10))]
    fed = {"a": [], "b": []}
    for _ in range(100):
        if not s.has_work():
            break
        before = {r.request_id: r.n_preempted for r in reqs}
        sched = s.schedule()
        for r in reqs:
            if r.n_preempted != before[r.request_id]:
                fed[r.request_id] = []              # its cache is gone: everything is fed again
        for e in sched:
            rid = e.request.request_id
            assert len(fed[rid]) == e.request.n_computed
            fed[rid] += e.tokens
            m.ensure(rid, e.request.n_computed + len(e.tokens))
            m.advance(rid, len(e.tokens))
        s.commit(sched, {e.request.request_id: 100 + len(e.request.output) for e in sched if e.sample})
    assert not s.has_work() and s.n_preemptions >= 1
    for r in reqs:
        assert fed[r.request_id] == (r.prompt + r.output)[:-1]


def test_portions_shrink_to_the_pages_that_are_free():
    m, s = mk(n_pages=6, page=4, slots=2, budget=32, chunk=32)
    s.add("a", list(range(12)), SamplingParams(max_tokens=4))
    run_step(m, s)                                   # a holds 3 pages (+1 when it decodes)
    s.add("b", list(range(20)), SamplingParams(max_tokens=1))
    sched, _ = run_step(m, s)
    got = {e.request.request_id: len(e.tokens) for e in sched}
    assert got["a"] == 1 and got["b"] == 8           # a takes its 4th page first; 2 pages = 8 tokens are left for b


def test_windowed_requests_may_be_longer_than_the_pool():
    m, s = mk(n_pages=6, page=4, slots=1, max_len=200, budget=8, chunk=8, window=6)
    r = s.add("a", list(range(100)), SamplingParams(max_tokens=50))
    for _ in range(400):
        if not s.has_work():
            break
        run_step(m, s)
    assert r.status == "finished" and len(r.output) == 50 and r.n_preempted == 0


def test_stop_tokens_and_eos():
    m, s = mk(eos_token_id=7)
    a = s.add("a", [1, 2], SamplingParams(max_tokens=10))
    b = s.add("b", [1, 2], SamplingParams(max_tokens=10, ignore_eos=True, stop_token_ids=(9,)))
    toks = iter([7, 7, 5, 9])
    run_step(m, s, token=lambda r: next(toks))       # a: 7 -> stop; b: 7 -> goes on
    assert a.finish_reason == "stop" and a.output == [7] and b.status == "running"
    run_step(m, s, token=lambda r: next(toks))
    run_step(m, s, token=lambda r: next(toks))
    assert b.finish_reason == "stop" and b.output == [7, 5, 9]


def test_length_limit_of_the_model():
    m, s = mk(max_len=10, n_pages=8)
    r = s.add("a", list(range(7)), SamplingParams(max_tokens=50))
    while s.has_work():
        run_step(m, s)
    assert r.finish_reason == "length" and len(r.prompt) + len(r.output) == 10


@pytest.mark.parametrize("seed", range(5))
def test_random_workloads_finish_and_keep_the_books(seed):
    rng = random.Random(seed)
    window = 7 if seed % 2 else 0
    m, s = mk(n_pages=10, page=4, slots=3, max_len=48, budget=12, chunk=rng.choice([3, 8, 12]), window=window)
    reqs = []
    pending = [(f"r{i}", rng.randint(1, 20), rng.randint(1, 12)) for i in range(14)]
    for _ in range(3000):
        if pending and rng.random() < 0.3:
            rid, plen, n_new = pending.pop()
            reqs.append((s.add(rid, [rng.randrange(50) for _ in range(plen)], SamplingParams(max_tokens=n_new)), n_new))
        if s.has_work():
            sched, _ = run_step(m, s)
            assert sched, "work waiting but nothing scheduled"
            assert sum(len(e.tokens) for e in sched) <= 12
            assert len({e.request.request_id for e in sched}) == len(sched)
        elif not pending:
            break
    assert not pending and not s.has_work()
    for r, n_new in reqs:
        assert r.status == "finished" and len(r.output) == n_new and r.output == [100 + i for i in range(n_new)]
    assert m.free_pages() == [10] and m.n_free_slots == 3


def test_abort_gives_everything_back():
    m, s = mk(slots=2)
    s.add("a", list(range(10)), SamplingParams(max_tokens=5))
    s.add("b", list(range(10)), SamplingParams(max_tokens=5))
    s.add("c", [1, 2], SamplingParams(max_tokens=5))
    run_step(m, s)
    assert s.abort("a") and s.abort("c") and not s.abort("zz")
    assert [r.request_id for r in s.running] == ["b"] and not s.waiting
    m.check_invariants()
    while s.has_work():
        run_step(m, s)
    assert m.free_pages() == [16] and m.n_free_slots == 2


def test_commit_in_two_halves_with_a_step_enqueued_in_between():
    """The engine enqueues step i + 1 before it has seen the tokens of step i: ``advance`` counts a
    token whose value is pending, ``resolve`` fills it in; a stop token found late ends the request
    and the token of the wasted step is dropped."""
    from flambeau_amd.engine.scheduler import PENDING
    m, s = mk(eos_token_id=7)
    a = s.add("a", [1, 2, 3], SamplingParams(max_tokens=4))
    b = s.add("b", [4, 5], SamplingParams(max_tokens=10))

    def enqueue():
        sched = s.schedule()
        for e in sched:
            m.ensure(e.request.request_id, e.request.n_computed + len(e.tokens))
            m.advance(e.request.request_id, len(e.tokens))
        s.advance(sched)
        return sched

    s1 = enqueue()                                       # prompts; both draw
    assert a.output == [PENDING] and b.output == [PENDING] and (a.pending_row, b.pending_row) == (0, 1)
    s2 = enqueue()                                       # decode rows fed from the device
    assert [e.tokens for e in s2] == [[PENDING], [PENDING]]
    assert s.resolve(s1, {"a": 11, "b": 7}) == [b]       # b drew the stop token in step 1
    assert b.output == [7] and b.finish_reason == "stop" and b not in s.running
    assert a.output == [11, PENDING]
    s3 = enqueue()                                       # only a is left
    assert [e.request.request_id for e in s3] == ["a"]
    assert s.resolve(s2, {"a": 12, "b": 99}) == []       # b's token of the wasted step is dropped
    assert b.output == [7] and a.output == [11, 12, PENDING]
    s4 = enqueue()                                       # a's fourth token: the length ends it at once
    assert a.status == "finished" and a not in s.running and m.n_free_slots == 3
    assert s.resolve(s3, {"a": 13}) == []                # not reported before its last token is known
    assert s.resolve(s4, {"a": 14}) == [a] and a.output == [11, 12, 13, 14] and a.finish_reason == "length"
    m.check_invariants()
    assert m.free_pages() == [16]


def test_any_of_several_end_of_sequence_ids_ends_a_request():
    m, s = mk(eos_token_id=(7, 11))
    a = s.add("a", [1, 2, 3], SamplingParams(max_tokens=10))
    b = s.add("b", [1, 2, 3], SamplingParams(max_tokens=10))
    c = s.add("c", [1, 2, 3], SamplingParams(max_tokens=4, ignore_eos=True))
    emits = {"a": [5, 11, 6], "b": [7], "c": [7, 11, 7, 11]}
    while s.has_work():
        run_step(m, s, token=lambda r: emits[r.request_id][len(r.output)])
    assert a.output == [5, 11] and a.finish_reason == "stop"
    assert b.output == [7] and b.finish_reason == "stop"
    assert c.output == [7, 11, 7, 11] and c.finish_reason == "length"
    assert m.free_pages() == [16] and m.n_free_slots == 3
    # one id, as before
    m, s = mk(eos_token_id=9)
    r = s.add("r", [1], SamplingParams(max_tokens=5))
    while s.has_work():
        run_step(m, s, token=lambda r: 9)
    assert r.output == [9]


def test_token_access_without_joining_prompt_and_output():
    from flambeau_amd.engine.scheduler import Request
    r = Request("x", [10, 11, 12], SamplingParams(), output=[20, 21])
    assert [r.token_at(i) for i in range(5)] == r.tokens
    for a in range(6):
        for b in range(a, 6):
            assert r.token_slice(a, b) == r.tokens[a:b]


def test_portions_are_cut_so_that_a_step_fills_whole_row_tiles():
    """Budget 520 (a portion of 512 beside 8 decoding requests), tiles of 128 rows: with 3 decode
    rows the portion is 509, so the step holds 512 rows; without a granule it is 512 + 3."""
    for granule, want in ((128, 509), (1, 512)):
        m = CacheManager([GroupSpec(1, 8, 0)], 400, 16, 9, 4096)
        s = Scheduler(m, max_batch_tokens=520, prefill_chunk_tokens=512, row_granule=granule)
        for rid in "abc":
            s.add(rid, [1, 2, 3], SamplingParams(max_tokens=50))
        run_step(m, s)
        s.add("long", list(range(2000)), SamplingParams(max_tokens=2))
        sched, _ = run_step(m, s)
        assert [(e.request.request_id, len(e.tokens)) for e in sched] == [("a", 1), ("b", 1), ("c", 1), ("long", want)]
    # a budget that holds less than a tile's worth of portions is left alone, and so is a short prompt
    m = CacheManager([GroupSpec(1, 8, 0)], 400, 16, 9, 4096)
    s = Scheduler(m, max_batch_tokens=100, prefill_chunk_tokens=64, row_granule=128)
    s.add("x", list(range(90)), SamplingParams(max_tokens=2))
    sched, _ = run_step(m, s)
    assert [len(e.tokens) for e in sched] == [64]
