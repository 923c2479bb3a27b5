"""The engine against the plain implementation, in 32-bit and in bfloat16, in every way of
cutting the work.  A difference that appears in one way of cutting only is a fault of the cache
or of the batch; the failure message names the first wrong position."""
import numpy as np
import pytest
import torch

import plain_model as pm
import replay_helpers as rh
from tiny_configs import TINY, write_sharpened

pytestmark = pytest.mark.gpu

STORE = {"float32": "float32", "bfloat16": "bfloat16"}
STORE_DTYPE = {"float32": torch.float32, "bfloat16": torch.bfloat16}
LENGTHS = {"A": [5, 12, 23, 40, 70, 97], "B": [1, 31, 97, 64, 129], "C": [3, 50, 33, 150, 81], "D": [4, 45, 100, 29, 160]}


def make_runner(model_dir, dtype, name, n_tokens, max_slots=8, page_size=None, tuned=True):
    from flambeau_amd.engine import ModelRunner, load_model
    ps = page_size or TINY[name]["page_size"]
    model, _ = load_model(model_dir, dtype=dtype, max_batch_tokens=512, tuned=tuned)
    runner = ModelRunner(model, n_pages=-(-n_tokens // ps), page_size=ps, max_slots=max_slots, max_logit_rows=512)
    # the cache starts full of NaN: a row that was never written, read by anyone, shows in the logits
    runner.storage.fill(float("nan"))
    return runner


def requests_for(name, seed=1):
    return rh.make_requests(TINY[name]["config"]["vocab_size"], LENGTHS[name], seed)


@pytest.fixture(scope="module")
def runners(model_dirs):
    """One runner per (configuration, dtype), with a pool so small that pages are used again."""
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            cache[(name, dtype)] = make_runner(model_dirs[(name, STORE[dtype])], dtype, name, n_tokens=448)
        return cache[(name, dtype)]
    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_cutting(model_dirs, runners, name, dtype, mode):
    d = model_dirs[(name, STORE[dtype])]
    reqs = requests_for(name)
    steps = {"whole": rh.trace_whole, "tail": rh.trace_tail, "portions": rh.trace_portions,
             "mixed": lambda r: rh.trace_mixed(r, seed=7)}[mode](reqs)
    runner = runners(name, dtype)
    got = rh.run_in_process(runner, steps)
    assert not runner.manager.live and runner.manager.free_pages() == [p.n_pages for p in runner.manager.pools]
    rh.compare(got, reqs, rh.plain_logits(d, reqs), dtype, f"{name} {mode}")
    if mode != "mixed":
        assert len(got) == sum(len(t) for t in reqs.values())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_peaked_attention_in_every_cutting(tmp_path_factory, name, dtype):
    """Queries and keys scaled up: single keys matter, so a key lost at a window's edge, at a
    page's edge or in a page that is used again moves the logits far beyond the tolerance.
    In bfloat16 the factor is smaller: scores of size 20 to 30 would turn the 8-bit rounding of
    queries and keys into errors of several percent in the softmax weights, whatever the engine
    does."""
    factor = 12.0 if dtype == "float32" else 4.0
    d = write_sharpened(name, tmp_path_factory.mktemp("sharp") / name, STORE[dtype], factor)
    reqs = rh.make_requests(TINY[name]["config"]["vocab_size"], [90, 41, 120, 66], seed=11)
    ref = rh.plain_logits(d, reqs)
    runner = make_runner(d, dtype, name, n_tokens=320)
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs)),
                        ("portions", rh.trace_portions(reqs, sizes=(3, 2, 9, 8, 2, 25, 7))),
                        ("mixed", rh.trace_mixed(reqs, seed=5, max_portion=19))]:
        got = rh.run_in_process(runner, steps)
        rh.compare(got, reqs, ref, dtype, f"peaked {name} {mode}")


def test_few_pages_are_used_again(model_dirs):
    """With room for little more than the live requests, later requests get the pages of earlier
    ones; their logits must not see what was there."""
    name, dtype = "B", "float32"
    d = model_dirs[(name, "float32")]
    reqs = rh.make_requests(384, [40, 40, 40, 40, 40, 40, 40, 40], seed=3)
    steps = rh.trace_mixed(reqs, seed=2, max_live=2, max_portion=16)
    runner = make_runner(d, dtype, name, n_tokens=rh.peak_tokens(steps, rounding=16))
    got = rh.run_in_process(runner, steps)
    rh.compare(got, reqs, rh.plain_logits(d, reqs), dtype, "reuse")
    pool = runner.manager.pools[0]
    assert pool.n_acquired >= 3 * pool.n_pages          # every page was handed out three times or more


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model_dirs, dtype):
    """A short prompt and 400 tokens one by one, past the window and over many pages."""
    name = "C"
    d = model_dirs[(name, STORE[dtype])]
    reqs = rh.make_requests(300, [420], seed=9)
    steps = rh.trace_tail(reqs, tail=400)
    runner = make_runner(d, dtype, name, n_tokens=448)
    got = rh.run_in_process(runner, steps)
    rh.compare(got, reqs, rh.plain_logits(d, reqs), dtype, "long decoding")
    # the window let pages go while the request was alive
    assert len(got) == 420


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(model_dirs, runners, name, dtype):
    """Prompts of one, two and three tokens: position 0 sees itself only."""
    d = model_dirs[(name, STORE[dtype])]
    reqs = rh.make_requests(TINY[name]["config"]["vocab_size"], [1, 2, 3], seed=21)
    runner = runners(name, dtype)
    ref = rh.plain_logits(d, reqs)
    rh.compare(rh.run_in_process(runner, rh.trace_whole(reqs)), reqs, ref, dtype, "first tokens whole")
    rh.compare(rh.run_in_process(runner, rh.trace_tail(reqs, tail=2)), reqs, ref, dtype, "first tokens one by one")


def test_logits_do_not_depend_on_neighbours(model_dirs, runners):
    """The same request alone and beside three others: bit for bit the same with the plain
    kernels of the 32-bit path (every row is reduced in a fixed order)."""
    name = "A"
    reqs = requests_for(name)
    runner = runners(name, "float32")
    alone = rh.run_in_process(runner, rh.trace_whole({"r3": reqs["r3"]}))
    steps = [dict(entries=[dict(id=r, tokens=reqs[r], want=list(range(len(reqs[r])))) for r in ("r1", "r3", "r0", "r4")],
                  end=["r1", "r3", "r0", "r4"])]
    together = rh.run_in_process(runner, steps)
    for p in range(len(reqs["r3"])):
        assert np.array_equal(alone[("r3", p)], together[("r3", p)])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wanted_rows_come_in_the_order_asked(model_dirs, runners, dtype):
    """``want`` may name every token of a step out of order, or one place twice: the rows come back in
    the order of the entries and of their ``want``, in eager steps and in captured decode steps."""
    name = "A"
    d = model_dirs[(name, STORE[dtype])]
    reqs = rh.make_requests(256, [2, 16, 9, 5], seed=31)
    ref = rh.plain_logits(d, reqs)
    runner = runners(name, dtype)
    perm = [int(i) for i in np.random.default_rng(4).permutation(16)]
    assert perm != sorted(perm)
    steps = [
        dict(entries=[dict(id="r0", tokens=reqs["r0"], want=[1, 0])], end=["r0"]),
        dict(entries=[dict(id="r0", tokens=reqs["r0"], want=[0, 0])], end=["r0"]),
        dict(entries=[dict(id="r0", tokens=reqs["r0"], want=[1, 1, 0, 1])], end=["r0"]),
        dict(entries=[dict(id="r1", tokens=reqs["r1"], want=perm)], end=["r1"]),
        # two requests whose wanted rows together cover every row of the step, out of order
        dict(entries=[dict(id="r2", tokens=reqs["r2"][:3], want=[2, 1, 0]), dict(id="r3", tokens=reqs["r3"][:2], want=[0, 1])], end=[]),
        # decode steps (captured): a place wanted twice, beside a request that wants nothing
        dict(entries=[dict(id="r2", tokens=[reqs["r2"][3]], want=[0, 0]), dict(id="r3", tokens=[reqs["r3"][2]], want=[])], end=[]),
        dict(entries=[dict(id="r3", tokens=[reqs["r3"][3]], want=[0, 0, 0]), dict(id="r2", tokens=[reqs["r2"][4]], want=[0])], end=["r2", "r3"]),
    ]
    from flambeau_amd.engine import StepEntry
    tol = rh.tolerance(dtype, max(float(np.abs(r).max()) for r in ref.values()))
    pos = {}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if e["id"] not in runner.manager.live:
                assert runner.begin(e["id"])
                pos[e["id"]] = 0
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        rows = runner.step(entries).cpu().double().numpy()
        expect = [(e["id"], pos[e["id"]] + w) for e in s["entries"] for w in e["want"]]
        assert rows.shape[0] == len(expect)
        for row, (rid, p) in zip(rows, expect):
            assert np.abs(row - ref[rid][p]).max() <= tol, (s, rid, p)
        for e in s["entries"]:
            pos[e["id"]] += len(e["tokens"])
        for rid in s["end"]:
            runner.end(rid)
    assert not runner.manager.live


def test_step_refuses_bad_batches(model_dirs, runners):
    from flambeau_amd.cache import CacheError
    from flambeau_amd.engine import StepEntry, StepError
    runner = runners("A", "float32")
    with pytest.raises(StepError, match="not live"):
        runner.step([StepEntry("x", [1])])
    assert runner.begin("x")
    with pytest.raises(StepError, match="twice"):
        runner.step([StepEntry("x", [1]), StepEntry("x", [2])])
    with pytest.raises(StepError, match="outside the vocabulary"):
        runner.step([StepEntry("x", [256])])
    with pytest.raises(StepError, match="wanted place"):
        runner.step([StepEntry("x", [1, 2], [2])])
    with pytest.raises(StepError, match="no tokens"):
        runner.step([StepEntry("x", [])])
    with pytest.raises(CacheError):
        runner.step([StepEntry("x", [1] * 129)])          # beyond max_position_embeddings = 128
    assert runner.cached_tokens("x") == 0                 # refused steps changed nothing
    runner.end("x")
    runner.manager.check_invariants()


# ---------------------------------------------------------------- generation through the entry point
def _plain_generate(d, prompt, n_new, temperature=0.0, seed=0, stop=(), **filters):
    cfg, w = pm.read_model_dir(d)
    rng = pm.Xoshiro(seed)
    toks, margins = list(prompt), []
    for _ in range(n_new):
        logits = pm.forward(cfg, w, toks)[-1].astype(np.float32)
        s = np.sort(logits)
        margins.append(float(s[-1] - s[-2]))
        toks.append(pm.sample(logits, rng, temperature=temperature, history=toks[len(prompt):], **filters))
        if toks[-1] in stop:
            break
    return toks[len(prompt):], margins


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(model_dirs, dtype):
    """Workload of the first tiny configuration: prompts of 5, 12, 23 and 40 tokens, 16 greedy
    tokens each, pages of 8, all four requests in flight with portions of 16."""
    from flambeau_amd import generate
    name = "A"
    d = model_dirs[(name, STORE[dtype])]
    prompts = list(rh.make_requests(256, [5, 12, 23, 40], seed=1).values())
    outs = generate(str(d), prompts, max_new_tokens=16, dtype=dtype, page_size=8, inflight_slots=4,
                    prefill_chunk_tokens=16, paged_kv=40)
    tie = 1e-4 if dtype == "float32" else 2e-2
    for prompt, out in zip(prompts, outs):
        want, margins = _plain_generate(d, prompt, 16)
        assert len(out) == 16
        for i, (a, b) in enumerate(zip(out, want)):
            if a != b:
                assert margins[i] < tie, f"token {i}: engine {a}, plain {b}, margin {margins[i]}"
                break


def test_temperature_generation_through_the_entry_point(model_dirs):
    """Workload of the second tiny configuration: prompts of 1, 31 and 97 tokens, 24 tokens each,
    one greedy and two at temperature 0.8 with seeded draws; pages of 16."""
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    d = model_dirs[("B", "float32")]
    prompts = list(rh.make_requests(384, [1, 31, 97], seed=3).values())
    temps, seeds = [0.0, 0.8, 0.8], [100, 101, 102]
    eng = LLMEngine.from_dir(str(d), EngineOptions(dtype="float32", page_size=16, inflight_slots=3,
                                                   prefill_chunk_tokens=32, paged_kv=24))
    outs = eng.generate(prompts, [SamplingParams(temperature=t, seed=s, max_tokens=24) for t, s in zip(temps, seeds)])
    for prompt, out, t, s in zip(prompts, outs, temps, seeds):
        want, _ = _plain_generate(d, prompt, 24, temperature=t, seed=s)
        assert out == want
    # the host sampler (filters) takes the same path through the scheduler
    outs2 = eng.generate(prompts[:2], [SamplingParams(temperature=0.8, top_k=384, seed=s, max_tokens=8) for s in seeds[:2]])
    for prompt, out, s in zip(prompts, outs2, seeds):
        assert out == _plain_generate(d, prompt, 8, temperature=0.8, seed=s, top_k=384)[0]
    assert not eng.runner.manager.live and eng.runner.manager.free_pages() == [24]


def test_a_request_s_tokens_do_not_depend_on_what_its_neighbours_ask_for(model_dirs):
    """A seeded temperature request beside a neighbour whose logits go to the host sampler (a top-k
    beyond what the device keeps) draws the tokens it draws alone, and the plain sampler's."""
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    d = model_dirs[("B", "float32")]
    prompts = list(rh.make_requests(384, [9, 14, 20], seed=23).values())
    eng = LLMEngine.from_dir(str(d), EngineOptions(dtype="float32", page_size=16, inflight_slots=3, prefill_chunk_tokens=32))
    mine = SamplingParams(temperature=0.8, seed=500, max_tokens=20)
    alone = eng.generate(prompts[:1], mine)[0]
    assert alone == _plain_generate(d, prompts[0], 20, temperature=0.8, seed=500)[0]
    beside = eng.generate(prompts, [mine, SamplingParams(temperature=0.9, top_k=7, seed=501, max_tokens=20),
                                    SamplingParams(temperature=0.0, repetition_penalty=1.3, top_k=3000, max_tokens=12)])
    assert not SamplingParams(top_k=3000).device_ok
    assert beside[0] == alone
    assert beside[1] == _plain_generate(d, prompts[1], 20, temperature=0.9, seed=501, top_k=7)[0]
    assert beside[2] == _plain_generate(d, prompts[2], 12, repetition_penalty=1.3, top_k=3000)[0]
    # and with the device sampler switched off everything goes through the host sampler
    host = LLMEngine.from_dir(str(d), EngineOptions(dtype="float32", page_size=16, inflight_slots=3, prefill_chunk_tokens=32,
                                                    gpu_sampler=False))
    greedy = SamplingParams(max_tokens=10)
    assert host.generate(prompts[:2], greedy) == eng.generate(prompts[:2], greedy)


def test_filtered_requests_stay_on_the_device(model_dirs, monkeypatch):
    """Top-k, top-p and min-p are drawn by the device sampler: no logits go to the host sampler (it
    raises here if called), the engine keeps a step in flight, and the tokens are the plain sampler's."""
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    import flambeau_amd.engine.llm as llm

    def no_host(*a, **k):
        raise AssertionError("the host sampler was called")
    monkeypatch.setattr(llm, "sample_host", no_host)
    d = model_dirs[("B", "float32")]
    prompts = list(rh.make_requests(384, [5, 23, 40, 12], seed=31).values())
    opts = [dict(temperature=0.9, top_k=12, seed=601), dict(temperature=0.7, top_p=0.8, seed=602),
            dict(temperature=1.2, top_k=50, top_p=0.95, min_p=0.05, seed=603), dict(temperature=1.0, min_p=0.2, seed=604)]
    eng = LLMEngine.from_dir(str(d), EngineOptions(dtype="float32", page_size=16, inflight_slots=4, prefill_chunk_tokens=32))
    seen_in_flight = []
    step = eng.step
    monkeypatch.setattr(eng, "step", lambda: (step(), seen_in_flight.append(eng._in_flight is not None))[0])
    outs = eng.generate(prompts, [SamplingParams(max_tokens=16, **o) for o in opts])
    assert any(seen_in_flight)
    for prompt, out, o in zip(prompts, outs, opts):
        assert out == _plain_generate(d, prompt, 16, **o)[0]


def test_penalties_and_bias_stay_on_the_device(model_dirs, monkeypatch):
    """Penalties over the generated tokens and a logit bias are applied on the device: the host
    sampler is never called (it raises here), a step stays in flight, and the tokens are the plain
    sampler's.  More requests than slots and so few pages that requests are pre-empted: a slot's
    row of counts passes from request to request and is counted anew for a request that returns."""
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    import flambeau_amd.engine.llm as llm

    def no_host(*a, **k):
        raise AssertionError("the host sampler was called")
    monkeypatch.setattr(llm, "sample_host", no_host)
    d = model_dirs[("B", "float32")]
    prompts = list(rh.make_requests(384, [5, 23, 40, 12, 9, 17], seed=37).values())
    opts = [dict(repetition_penalty=1.8), dict(temperature=0.8, presence_penalty=0.7, frequency_penalty=0.3, seed=611),
            dict(logit_bias={3: 4.0, 200: 2.5, 9999: 1.0}), dict(temperature=0.9, repetition_penalty=0.7, top_k=20, seed=613),
            dict(temperature=1.1, frequency_penalty=1.5, logit_bias={7: -3.0, 11: 6.0}, min_p=0.02, seed=614),
            dict(temperature=0.7, seed=615)]
    eng = LLMEngine.from_dir(str(d), EngineOptions(dtype="float32", page_size=16, inflight_slots=3, prefill_chunk_tokens=32,
                                                   paged_kv=6))
    seen_in_flight = []
    step = eng.step
    monkeypatch.setattr(eng, "step", lambda: (step(), seen_in_flight.append(eng._in_flight is not None))[0])
    n_new = 24
    outs = eng.generate(prompts, [SamplingParams(max_tokens=n_new, **o) for o in opts])
    assert any(seen_in_flight) and eng.scheduler.n_preemptions > 0
    for prompt, out, o in zip(prompts, outs, opts):
        assert out == _plain_generate(d, prompt, n_new, **o)[0], o
    assert not eng.runner.manager.live


def test_the_sampler_s_history_follows_a_request_through_slots():
    """A request that is pre-empted comes back in whatever slot is free: its row of token counts is
    taken over when it kept drawing in the same slot and counted anew otherwise, also when it returns
    to a slot whose row still holds its counts from before it drew tokens elsewhere."""
    from flambeau_amd import SamplingParams
    from flambeau_amd.sampling.device import DeviceSampler
    from flambeau_amd.sampling.host import penalised
    V = 50
    sampler = DeviceSampler(torch.device("cuda:0"), 4)
    rng = np.random.default_rng(3)
    p = SamplingParams(repetition_penalty=1.5, presence_penalty=0.3, frequency_penalty=0.2)

    class Req:
        def __init__(self): self.output = []
    a, b = Req(), Req()
    for slot, req, counted_anew in [(0, a, True), (0, a, False), (1, b, True), (2, a, True), (2, a, False), (0, a, True),
                                    (0, a, False), (1, b, False), (0, b, True), (2, a, True)]:
        logits = rng.normal(0, 2, (1, V)).astype(np.float32)
        assert sampler.holds_history(slot, req, len(req.output)) == (not counted_anew)
        tok = sampler.sample(torch.tensor(logits, device="cuda:0"), [0.0], [0.0], None, [(slot, req, req.output, *p.penalties)])[0]
        assert tok == int(np.argmax(penalised(logits[0], p, req.output)))
        req.output.append(tok)
        assert sampler._counts[slot].cpu().numpy().tolist() == np.bincount(req.output, minlength=V).tolist()
    assert len(a.output) == 7 and len(b.output) == 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_stop_tokens_end_requests_while_the_next_step_is_in_flight(model_dirs, dtype):
    """The engine runs one step ahead of the host: when a stop id (or one of several end-of-sequence
    ids) arrives, the step after it is already enqueued.  Its token is dropped, the pages come back,
    and the other requests' tokens are what they are alone.  Pages are so few that requests are
    pre-empted on the way."""
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    d = model_dirs[("D", STORE[dtype])]          # config.json names the end-of-sequence ids 7 and 11
    prompts = list(rh.make_requests(210, [6, 17, 30, 11], seed=41).values())
    n_new = 24
    free = [_plain_generate(d, p, n_new)[0] for p in prompts]
    # stop ids: a token the first request emits in the middle, one the third emits early
    stops = (free[0][9], free[2][3])
    want = []
    for out in free:
        cut = next((i for i, t in enumerate(out) if t in stops or t in (7, 11)), len(out) - 1)
        want.append(out[:cut + 1])
    assert any(len(w) < n_new for w in want)
    eng = LLMEngine.from_dir(str(d), EngineOptions(dtype=dtype, page_size=8, inflight_slots=3, prefill_chunk_tokens=16,
                                                   paged_kv=7))
    got = eng.generate(prompts, SamplingParams(max_tokens=n_new, stop_token_ids=stops))
    if dtype == "float32":
        assert got == want
    else:
        # rounding may move a near-tie, so the tokens are not compared; every output still ends at its
        # first stop or end-of-sequence id, or at the length
        for g in got:
            assert len(g) == n_new or g[-1] in stops or g[-1] in (7, 11)
            assert not any(t in stops or t in (7, 11) for t in g[:-1])
    assert not eng.runner.manager.live and eng.runner.manager.free_pages() == [7, 7]
    eng.runner.manager.check_invariants()
    if dtype == "float32":
        assert eng.scheduler.n_preemptions > 0
        # ignore_eos lets a request run past an end-of-sequence id, not past a stop id
        again = eng.generate(prompts[:1], SamplingParams(max_tokens=n_new, ignore_eos=True, stop_token_ids=stops))
        cut = min(i for i, t in enumerate(free[0]) if t in stops)
        assert again[0] == free[0][:cut + 1]


def test_generation_survives_preemption(model_dirs):
    """So few pages that running requests are pre-empted and recomputed: the tokens stay the same."""
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    d = model_dirs[("B", "float32")]
    prompts = list(rh.make_requests(384, [30, 30, 30], seed=4).values())
    roomy = LLMEngine.from_dir(str(d), EngineOptions(dtype="float32", inflight_slots=3, paged_kv=24, prefill_chunk_tokens=64))
    want = roomy.generate(prompts, SamplingParams(max_tokens=30))
    tight = LLMEngine.from_dir(str(d), EngineOptions(dtype="float32", inflight_slots=3, paged_kv=8, prefill_chunk_tokens=64))
    got = tight.generate(prompts, SamplingParams(max_tokens=30))
    assert tight.scheduler.n_preemptions > 0
    assert got == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_equal_eager_ones(model_dirs, dtype):
    """Steps of single tokens replay a captured graph per batch-size bucket.  Every replay, with
    eager steps and synchronisations between them, gives the logits of the eager step."""
    name = "A"
    d = model_dirs[(name, STORE[dtype])]
    reqs = rh.make_requests(256, [30, 45, 37], seed=17)
    from flambeau_amd.engine import ModelRunner, load_model
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=256)
    results = []
    for graphs in (False, True):
        runner = ModelRunner(model, n_pages=32, page_size=8, max_slots=4, max_logit_rows=256, decode_graphs=graphs)
        assert runner.decode_graphs == graphs
        steps = []
        # prompts in portions, then decode rows of 3, 2 and 1 requests (buckets 4, 2, 1), with a
        # portion of another request between replays
        steps.append(dict(entries=[dict(id=r, tokens=reqs[r][:20], want=[19]) for r in reqs], end=[]))
        for i in range(20, 30):
            steps.append(dict(entries=[dict(id=r, tokens=[reqs[r][i]], want=[0]) for r in reqs], end=["r0"] if i == 29 else []))
        steps.append(dict(entries=[dict(id="r1", tokens=reqs["r1"][30:34], want=[0, 3])], end=[]))
        for i in range(30, 37):
            e = [dict(id="r2", tokens=[reqs["r2"][i]], want=[0])]
            if i + 4 < 45:
                e.append(dict(id="r1", tokens=[reqs["r1"][i + 4]], want=[] if i % 2 else [0]))
            steps.append(dict(entries=e, end=[]))
        steps.append(dict(entries=[dict(id="r1", tokens=[reqs["r1"][41]], want=[0])], end=["r1", "r2"]))
        results.append(rh.run_in_process(runner, steps))
        if graphs:
            assert sorted({bucket for bucket, _ in runner._graphs}) == [1, 2, 4]
    eager, graphed = results
    assert eager.keys() == graphed.keys() and len(eager) > 30
    for k in eager:
        assert np.array_equal(eager[k], graphed[k]), k
    rh.compare(graphed, reqs, rh.plain_logits(d, reqs), dtype, "captured steps")


def test_a_bucket_has_a_graph_for_each_thing_the_mixers_decide(model_dirs):
    """While no row's keys are split the kernel that merges splits is left out of the step; when a
    context grows beyond what one split holds the same bucket gets a second graph with it.  Both give
    the eager step's logits, before and after the change, and the plain implementation's."""
    d = model_dirs[("B", "bfloat16")]
    reqs = rh.make_requests(384, [230, 60], seed=23)
    from flambeau_amd.engine import ModelRunner, load_model
    model, _ = load_model(d, dtype="bfloat16", max_batch_tokens=256)
    steps = [dict(entries=[dict(id="r0", tokens=reqs["r0"][:90], want=[89]), dict(id="r1", tokens=reqs["r1"][:20], want=[])], end=[])]
    for i in range(90, 230):                       # r0 passes 128 keys on the way; r1 decodes beside it for a while
        e = [dict(id="r0", tokens=[reqs["r0"][i]], want=[0])]
        if i - 70 < 60:
            e.append(dict(id="r1", tokens=[reqs["r1"][i - 70]], want=[0]))
        steps.append(dict(entries=e, end=["r1"] if i - 70 == 59 else []))
    steps[-1]["end"] = ["r0"]
    results = []
    for graphs in (False, True):
        runner = ModelRunner(model, n_pages=24, page_size=16, max_slots=2, max_logit_rows=256, decode_graphs=graphs,
                             step_programs=False)
        runner.storage.fill(float("nan"))
        results.append(rh.run_in_process(runner, steps))
        if graphs:
            by_bucket = {}
            for bucket, decided in runner._graphs:
                by_bucket.setdefault(bucket, set()).add(decided)
            assert set(by_bucket) == {1, 2} and len(by_bucket[2]) == 2, by_bucket          # (r0 is alone only once it is split)
    eager, graphed = results
    assert eager.keys() == graphed.keys() and len(eager) > 170
    for k in eager:
        assert np.array_equal(eager[k], graphed[k]), k
    rh.compare(graphed, reqs, rh.plain_logits(d, reqs), "bfloat16", "graphs with and without the kernel that merges")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_steps_equal_eager_ones(model_dirs, dtype):
    """Steps that hold prompt portions are recorded while they run and replayed from native code when
    a step of the same shape comes again.  Every replay, for other requests, contexts and pages than
    the recording saw, gives bit for bit what the step gives when Python launches it."""
    name = "D"                                        # two cache groups: two block tables in the metadata
    d = model_dirs[(name, STORE[dtype])]
    reqs = rh.make_requests(210, [70, 70, 70, 31, 31, 150], seed=27)
    from flambeau_amd.engine import ModelRunner, load_model
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=256)
    assert model.replayable()
    portions = rh.trace_portions(reqs, sizes=(16, 9, 16, 2, 16, 9))          # the same sizes again and again
    mixed = rh.trace_mixed(reqs, seed=4, max_portion=12)
    results = []
    for programs in (False, True):
        runner = ModelRunner(model, n_pages=40, page_size=8, max_slots=4, max_logit_rows=256, step_programs=programs,
                             decode_graphs=False)
        runner.storage.fill(float("nan"))
        got = rh.run_in_process(runner, portions)
        got2 = rh.run_in_process(runner, mixed)
        results.append((got, got2))
        if programs:
            assert runner.n_replayed > 20
            # a longer step than any before makes buffers grow: programs recorded on the old ones are
            # not replayed, and the steps after it are right
            before = runner.n_recorded
            big = {"big": rh.make_requests(210, [200], seed=5)["r0"]}
            ref_big = rh.plain_logits(d, big)
            rh.compare(rh.run_in_process(runner, rh.trace_whole(big)), big, ref_big, dtype, "after growth: whole")
            again = rh.run_in_process(runner, portions)
            assert runner.n_recorded > before + 3
            for k in got:
                assert np.array_equal(again[k], got[k]), k
        else:
            assert runner.n_replayed == 0 and runner.n_recorded == 0
    (eager, eager2), (replayed, replayed2) = results
    assert eager.keys() == replayed.keys() and eager2.keys() == replayed2.keys()
    for k in eager:
        assert np.array_equal(eager[k], replayed[k]), k
    for k in eager2:
        assert np.array_equal(eager2[k], replayed2[k]), k
    rh.compare(replayed, reqs, rh.plain_logits(d, reqs), dtype, "recorded steps")


def test_a_block_that_cannot_be_recorded_runs_between_recorded_stretches(model_dirs, tmp_path):
    """One block of the model says that its launches cannot be recorded (as a block with a part that
    calls torch would): steps are still recorded, in stretches, and the block runs again between them at
    every replay, with that step's requests and pages.  Logits agree with the plain implementation
    and, but for the add and the norm around the block that are not fused then, with the unrecorded
    engine."""
    import json, shutil
    from flambeau_amd.config.mistral import MistralConfig
    from flambeau_amd.engine import ModelRunner, load_model
    from flambeau_amd.kernels.library import Program
    from flambeau_amd.models.decoder import LayerSpec
    from flambeau_amd.models.mistral import mistral_spec
    from flambeau_amd.parts import BLOCKS, PartSpec
    from flambeau_amd.parts.block import PreNormBlock
    from flambeau_amd.registry import register_architecture
    if "prenorm_unrecorded" not in BLOCKS.known():
        @BLOCKS.register("prenorm_unrecorded")
        class Unrecorded(PreNormBlock):
            replayable = False

        def spec(cfg):
            m = mistral_spec(cfg)
            m.layers[1] = LayerSpec(PartSpec("prenorm_unrecorded", m.layers[1].block.params), m.layers[1].names)
            return m
        register_architecture("MistralOneBlockUnrecorded", MistralConfig, spec)
    dtype = "bfloat16"
    src = model_dirs[("D", STORE[dtype])]
    d = tmp_path / "model"
    shutil.copytree(src, d)
    raw = json.loads((d / "config.json").read_text())
    raw["architectures"] = ["MistralOneBlockUnrecorded"]
    (d / "config.json").write_text(json.dumps(raw))
    reqs = rh.make_requests(210, [70, 70, 31, 31, 150], seed=29)
    ref = rh.plain_logits(src, reqs)
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=256)
    assert model.replayable() and not model._part_replayable(model.blocks[1])
    runner = ModelRunner(model, n_pages=40, page_size=8, max_slots=4, max_logit_rows=256, decode_graphs=False)
    runner.storage.fill(float("nan"))
    portions = rh.trace_portions(reqs, sizes=(16, 9, 16, 2, 16, 9))
    got = rh.run_in_process(runner, portions)
    got2 = rh.run_in_process(runner, rh.trace_mixed(reqs, seed=6, max_portion=12))
    assert runner.n_replayed > 20
    kinds = [[isinstance(s, Program) for s in r.stretches] for r in runner._programs.values()]
    assert kinds and all(k == [True, False, True] for k in kinds)          # launches, the block, launches
    rh.compare(got, reqs, ref, dtype, "one unrecorded block: portions")
    rh.compare(got2, reqs, ref, dtype, "one unrecorded block: mixed")
    # A stretch that keeps coming back becomes a device graph of its own, the block still runs between
    # the graphs: steps of single tokens of this model, which cannot be captured whole, replay two graphs
    # around one block run from Python.
    runner = ModelRunner(model, n_pages=40, page_size=8, max_slots=4, max_logit_rows=256)
    assert not runner.decode_graphs and runner.step_programs
    runner.storage.fill(float("nan"))
    got3 = rh.run_in_process(runner, rh.trace_tail(reqs, tail=32))
    graphed = [r for r in runner._programs.values() if r.graphs]
    assert graphed and all(sorted(r.graphs) == [0, 2] for r in graphed)
    assert max(r.hits for r in graphed) > 10
    rh.compare(got3, reqs, ref, dtype, "one unrecorded block: single tokens through graphs of stretches")


@pytest.fixture(scope="module")
def wide_model_dir(tmp_path_factory):
    """Two layers with the layer sizes of a 7B model (width 4096, 32 heads in 8 groups of 128,
    feed-forward 14336, vocabulary 32768), written by the random-weights mode."""
    import torch
    from flambeau_amd.weights import write_random_model
    config = {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_act": "silu",
              "num_hidden_layers": 2, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8,
              "intermediate_size": 14336, "vocab_size": 32768, "rope_theta": 1e6, "sliding_window": None,
              "rms_norm_eps": 1e-5, "max_position_embeddings": 32768, "tie_word_embeddings": False}
    return write_random_model(config, tmp_path_factory.mktemp("wide") / "model", seed=7, std=0.02, gain_std=0.01,
                              store_dtype=torch.bfloat16)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cutting_at_real_layer_sizes(wide_model_dir, dtype):
    """The sizes the kernels are tuned for (and the kernels that only those sizes reach: the tiled
    products with their fusions, many heads, pages of 16 under long rows), in portions and mixed."""
    from flambeau_amd.engine import ModelRunner, load_model
    reqs = rh.make_requests(32768, [150, 40, 90], seed=11)
    model, _ = load_model(wide_model_dir, dtype=dtype, max_batch_tokens=512)
    runner = ModelRunner(model, n_pages=24, page_size=16, max_slots=4, max_logit_rows=512)
    runner.storage.fill(float("nan"))
    ref = rh.plain_logits(wide_model_dir, reqs)
    for what, steps in (("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=12)),
                        ("portions", rh.trace_portions(reqs, sizes=(2, 70, 3, 17, 2, 130, 31, 4))),
                        ("mixed", rh.trace_mixed(reqs, seed=3, max_portion=90))):
        got = rh.run_in_process(runner, steps)
        assert not runner.manager.live
        rh.compare(got, reqs, ref, dtype, f"wide {what}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_short_portions_behind_a_long_context(tmp_path_factory, dtype):
    """A request of 2,000 tokens in portions that shrink: the late portions give the tiled attention
    few tiles with many keys, which it then splits over blocks and merges."""
    import torch
    from flambeau_amd.engine import ModelRunner, load_model
    from flambeau_amd.kernels import tuned
    from flambeau_amd.weights import write_random_model
    config = {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_act": "silu",
              "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
              "intermediate_size": 96, "vocab_size": 150, "rope_theta": 1e4, "sliding_window": None,
              "rms_norm_eps": 1e-5, "max_position_embeddings": 2048, "tie_word_embeddings": False}
    d = write_random_model(config, tmp_path_factory.mktemp("long") / "model", seed=12, std=0.08, gain_std=0.02,
                           store_dtype=STORE_DTYPE[dtype])
    assert tuned.attn_prefill_splits(2, 4, 2, 16, 1900) > 1
    reqs = rh.make_requests(150, [2000], seed=9)
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=1024)
    runner = ModelRunner(model, n_pages=140, page_size=16, max_slots=2, max_logit_rows=1024)
    runner.storage.fill(float("nan"))
    steps = rh.trace_portions(reqs, sizes=(1000, 700, 100, 64, 9, 70, 30, 27))
    got = rh.run_in_process(runner, steps)
    rh.compare(got, reqs, rh.plain_logits(d, reqs), dtype, "long context")


def test_context_beyond_65536_tokens(tmp_path, monkeypatch):
    """70,000 tokens of context (4,375 pages of 16: block tables 8,192 wide from token 65,537 on): the
    prompt in portions of 4,096, the last tokens one by one, against the plain implementation at rows of
    the last two portions and at every decoded token.  The first layer has a window of 700 (so the plain
    implementation needs no score matrix of 70,000 squared there), the second sees everything and is
    computed at the wanted rows only.  In bfloat16 the tiled and the split-K attention kernels must take
    tables this wide themselves: the plain attention kernel is not allowed to run."""
    import torch
    from flambeau_amd.engine import ModelRunner, load_model
    from flambeau_amd.kernels import ops, tuned
    from flambeau_amd.weights import write_random_model
    config = {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_act": "silu",
              "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
              "intermediate_size": 96, "vocab_size": 150, "rope_theta": 1e6, "sliding_window": 700,
              "layer_types": ["sliding_attention", "full_attention"],
              "rms_norm_eps": 1e-5, "max_position_embeddings": 131072, "tie_word_embeddings": False}
    d = write_random_model(config, tmp_path / "model", seed=14, std=0.08, gain_std=0.02, store_dtype=torch.bfloat16)
    n, tail = 70000, 6
    toks = rh.make_requests(150, [n], seed=10)["r0"]
    steps, wanted, at = [], [], 0
    while at < n - tail:
        cnt = min(4096, n - tail - at)
        # rows of the portions that lie beyond 65,536 tokens: tile edges, and the portion's last rows
        want = sorted({0, 63, 64, 1000, 2047, cnt - 2, cnt - 1} & set(range(cnt))) if at + cnt > 65536 else []
        steps.append(dict(step=len(steps), entries=[dict(id="r0", tokens=toks[at:at + cnt], want=want)], end=[]))
        wanted += [at + r for r in want]
        at += cnt
    for i in range(n - tail, n):
        steps.append(dict(step=len(steps), entries=[dict(id="r0", tokens=toks[i:i + 1], want=[0])], end=["r0"] if i == n - 1 else []))
        wanted.append(i)
    assert len(wanted) == 12 + tail and min(wanted) == 65536
    cfg, w = pm.read_model_dir(d)
    ref = dict(zip(wanted, pm.forward(cfg, w, toks, rows=wanted)))
    scale = max(float(np.abs(v).max()) for v in ref.values())
    for dtype in ("float32", "bfloat16"):
        widths = []
        if dtype == "bfloat16":
            def no_plain(*a, **k):
                raise AssertionError("the plain attention kernel ran on the bfloat16 path")
            monkeypatch.setattr(ops, "attn_plain", no_plain)
            tiled = tuned.attn_prefill

            def counted(q, out, cache, tiles, positions, table, *a, **k):
                widths.append(table.shape[1])
                return tiled(q, out, cache, tiles, positions, table, *a, **k)
            monkeypatch.setattr(tuned, "attn_prefill", counted)
        model, _ = load_model(d, dtype=dtype, max_batch_tokens=4096)
        runner = ModelRunner(model, n_pages=4400, page_size=16, max_slots=2, max_logit_rows=8)
        runner.storage.fill(float("nan"))
        got = rh.run_in_process(runner, steps)
        assert not runner.manager.live and runner.manager.free_pages() == [4400, 4400]
        del runner, model
        torch.cuda.empty_cache()
        assert sorted(p for _, p in got) == wanted
        tol = 1e-4 if dtype == "float32" else 2e-2 * scale
        for (_, p), row in got.items():
            assert np.isfinite(row).all() and np.abs(row - ref[p]).max() <= tol, (dtype, p, np.abs(row - ref[p]).max())
        if dtype == "bfloat16":
            assert 8192 in widths, widths          # both layers of the two widest portions


def test_serving_loop_under_random_pressure(model_dirs):
    """Random mixes of requests, slots, pages, portion sizes, sampling and stop ids through the serving
    loop (which runs a step ahead of the host and pre-empts when pages run out): every request's
    tokens are those it gets alone, whatever happens around it, and no page or slot is lost."""
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    from flambeau_amd.engine import load_model
    n_pre = n_stopped = 0
    for name, ps in (("A", 8), ("D", 8), ("B", 16)):
        d = model_dirs[(name, "float32")]
        vocab = TINY[name]["config"]["vocab_size"]
        ctx = min(TINY[name]["config"]["max_position_embeddings"], 256)
        model, _ = load_model(d, dtype="float32", max_batch_tokens=ctx + 8)
        alone = LLMEngine(model, EngineOptions(dtype="float32", inflight_slots=1, prefill_chunk_tokens=ctx, page_size=ps, ctx_cap=ctx))
        for case in range(40):
            rng = np.random.default_rng(1000 * ps + case)
            n_req = int(rng.integers(3, 8))
            new = int(rng.integers(4, 30))
            prompts = [[int(t) for t in rng.integers(0, vocab, int(rng.integers(1, ctx - new - 1)))] for _ in range(n_req)]
            temp = float(rng.choice([0.0, 0.0, 0.8]))
            stops = tuple(int(t) for t in rng.integers(0, vocab, int(rng.integers(0, 12))))
            params = [SamplingParams(max_tokens=new, temperature=temp, seed=100 + i, stop_token_ids=stops) for i in range(n_req)]
            want = [alone.generate([p], sp)[0] for p, sp in zip(prompts, params)]
            longest = -(-(max(len(p) for p in prompts) + new) // ps)
            slots = int(rng.integers(2, 6))
            pages = longest + int(rng.integers(1, 2 * longest))
            chunk = int(rng.choice([16, 64, ctx]))
            eng = LLMEngine(model, EngineOptions(dtype="float32", inflight_slots=slots, prefill_chunk_tokens=chunk, page_size=ps,
                                                 paged_kv=pages, ctx_cap=ctx, max_batch_tokens=ctx + 8))
            got = eng.generate(prompts, params)
            what = f"{name} case {case}: slots {slots}, pages {pages}, portions {chunk}, temperature {temp}, {len(stops)} stop ids"
            assert got == want, what
            assert not eng.runner.manager.live and all(f == pages for f in eng.runner.manager.free_pages()), what
            eng.runner.manager.check_invariants()
            n_pre += eng.scheduler.n_preemptions
            n_stopped += sum(len(g) < new for g in got)
    assert n_pre > 0 and n_stopped > 0          # the cases did pre-empt, and did stop requests early


def test_arrivals_and_aborts_while_a_step_is_in_flight(model_dirs):
    """Requests that arrive while others decode, and aborts at random steps (of waiting requests, of
    requests in the middle of their prompt, of requests whose last token the host has not seen yet),
    through the serving loop with tight pools: a surviving request's tokens are those it gets alone, an
    aborted request's tokens so far are a prefix of those, and every page and slot comes back.  (The
    reference checks the same of its sessions: crates/forward/tests/multi_session_leak.rs:180-193;
    requests join its running batch in crates/server/src/routes.rs:631-733.)"""
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    from flambeau_amd.engine import load_model
    from flambeau_amd.engine.scheduler import PENDING
    seen = dict(pending=0, waiting=0, prompt=0, joined=0, preempted=0, survivors=0)
    for name, ps in (("A", 8), ("D", 8)):
        d = model_dirs[(name, "float32")]
        vocab = TINY[name]["config"]["vocab_size"]
        ctx = min(TINY[name]["config"]["max_position_embeddings"], 200)
        model, _ = load_model(d, dtype="float32", max_batch_tokens=ctx + 8)
        alone = LLMEngine(model, EngineOptions(dtype="float32", inflight_slots=1, prefill_chunk_tokens=ctx, page_size=ps, ctx_cap=ctx))
        for case in range(25):
            rng = np.random.default_rng(7000 + 100 * ps + case + (500 if name == "D" else 0))
            n_req = int(rng.integers(4, 9))
            new = int(rng.integers(6, 30))
            prompts = [[int(t) for t in rng.integers(0, vocab, int(rng.integers(1, ctx - new - 1)))] for _ in range(n_req)]
            stops = tuple(int(t) for t in rng.integers(0, vocab, int(rng.integers(0, 6))))
            params = [SamplingParams(max_tokens=new, temperature=float(rng.choice([0.0, 0.8])), seed=300 + i,
                                     top_k=int(rng.integers(2, 40)) if rng.random() < 0.3 else None,
                                     repetition_penalty=1.3 if rng.random() < 0.2 else 1.0, stop_token_ids=stops)
                      for i in range(n_req)]
            want = [alone.generate([p], sp)[0] for p, sp in zip(prompts, params)]
            longest = -(-(max(len(p) for p in prompts) + new) // ps)
            slots = int(rng.integers(2, 5))
            pages = longest + int(rng.integers(1, 2 * longest))
            chunk = int(rng.choice([16, 64, ctx]))
            eng = LLMEngine(model, EngineOptions(dtype="float32", inflight_slots=slots, prefill_chunk_tokens=chunk, page_size=ps,
                                                 paged_kv=pages, ctx_cap=ctx, max_batch_tokens=ctx + 8))
            arrive = sorted(int(a) for a in rng.integers(0, 25, n_req))
            arrive[0] = 0
            kill = {i: int(rng.integers(a, a + 30)) for i, a in enumerate(arrive) if rng.random() < 0.4}
            reqs, aborted, step_no = {}, set(), 0
            what = f"{name} case {case}: slots {slots}, pages {pages}, portions {chunk}"
            while len(reqs) < n_req or eng.has_work():
                for i, a in enumerate(arrive):
                    if a == step_no:
                        seen["joined"] += any(r.status == "running" and r.output for r in reqs.values())
                        reqs[i] = eng.add_request(prompts[i], params[i], request_id=f"r{i}")
                for i, k in kill.items():
                    if k == step_no and i in reqs and reqs[i].status != "finished":
                        r = reqs[i]
                        seen["pending"] += PENDING in r.output
                        seen["waiting"] += r.status == "waiting"
                        seen["prompt"] += r.status == "running" and not r.output
                        assert eng.abort(f"r{i}"), what
                        assert r.status == "finished" and r.finish_reason == "abort"
                        aborted.add(i)
                if eng.has_work():
                    eng.step()
                step_no += 1
                assert step_no < 3000, what
            eng.flush()
            eng.runner.manager.check_invariants()
            assert not eng.runner.manager.live and all(f == pages for f in eng.runner.manager.free_pages()), what
            assert eng.runner.manager.n_free_slots == slots, what
            seen["preempted"] += eng.scheduler.n_preemptions
            for i in range(n_req):
                out = [t for t in reqs[i].output if t != PENDING]
                if i in aborted:
                    assert out == want[i][:len(out)], f"{what}: the tokens of aborted request {i} differ"
                else:
                    seen["survivors"] += 1
                    assert list(reqs[i].output) == want[i], f"{what}: request {i} differs (aborted: {sorted(aborted)})"
            assert not eng.abort("r0") and not eng.abort("nobody")          # finished or unknown: nothing to drop
    assert all(v > 0 for v in seen.values()), seen
