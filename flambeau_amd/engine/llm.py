"""The engine a user holds: model + cache + step function + scheduler + sampler.

``LLMEngine.generate`` runs the single scheduling loop until every request has finished:
``while work: batch = schedule(); logits = step(batch); sample; commit``.  Token ids go in,
token ids come out (there is no tokenizer here)."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..sampling.device import DeviceSampler
from ..sampling.host import sample_host
from ..sampling.params import SamplingParams
from .loading import load_model, random_model
from .scheduler import Request, Scheduler
from .step import ModelRunner, StepEntry


@dataclass
class EngineOptions:
    """Sizing knobs.  Names follow the reference's serve flags where it has them
    (crates/cli/src/main.rs:124-218): ``inflight_slots`` (requests running at a time),
    ``prefill_chunk_tokens``, ``paged_kv`` (pages in the pool, 16 tokens each by default),
    ``max_queue_depth``, ``ctx_cap`` (clamps the model's maximum length), ``gpu_sampler``."""
    dtype: str = "bfloat16"
    device: str = "cuda:0"
    inflight_slots: int = 4
    prefill_chunk_tokens: int = 512
    max_batch_tokens: int | None = None     # tokens per step; default prefill_chunk_tokens + inflight_slots
    row_granule: int | None = None          # steps of many rows hold a multiple of this many; default: the kernels' row tile
    paged_kv: int | None = None             # pages; default: enough for inflight_slots * ctx
    page_size: int = 16
    max_queue_depth: int = 0
    ctx_cap: int | None = None
    gpu_sampler: bool = True
    tuned_kernels: bool = True
    decode_graphs: bool = True
    seed: int = 0


class LLMEngine:
    def __init__(self, model, options: EngineOptions | None = None):
        self.options = opt = options or EngineOptions()
        self.model = model
        spec = model.spec
        ctx = min(opt.ctx_cap or spec.max_position, spec.max_position)
        n_pages = opt.paged_kv or opt.inflight_slots * -(-ctx // opt.page_size)
        self.runner = ModelRunner(model, n_pages=n_pages, page_size=opt.page_size, max_slots=opt.inflight_slots,
                                  max_seq_len=ctx, max_logit_rows=max(opt.inflight_slots, 1),
                                  decode_graphs=opt.decode_graphs)
        self.scheduler = Scheduler(self.runner.manager, max_batch_tokens=model.rt.max_batch_tokens,
                                   prefill_chunk_tokens=opt.prefill_chunk_tokens,
                                   max_queue_depth=opt.max_queue_depth,
                                   eos_token_id=getattr(spec, "eos_token_ids", ()) or spec.eos_token_id,
                                   default_seed=opt.seed,
                                   row_granule=opt.row_granule or model.rt.row_granule)
        self.sampler = DeviceSampler(model.rt.device, max(opt.inflight_slots, 1), vocab_size=spec.vocab_size)
        # tokens drawn on the device are fed to the next step on the device: the host enqueues
        # step i + 1 while step i runs and reads step i's tokens afterwards
        self.runner.token_feedback = self.sampler.ids
        self._in_flight = None            # (scheduled, sampler handle) of the step the host has not read yet
        self._pick_host = self._pick_dev = None
        self._next_id = 0

    @classmethod
    def from_dir(cls, model_dir, options: EngineOptions | None = None):
        opt = options or EngineOptions()
        mbt = opt.max_batch_tokens or (opt.prefill_chunk_tokens + opt.inflight_slots)
        model, _ = load_model(model_dir, dtype=opt.dtype, device=opt.device, max_batch_tokens=mbt,
                              tuned=opt.tuned_kernels)
        return cls(model, opt)

    # ------------------------------------------------------------ requests
    def add_request(self, prompt, params: SamplingParams | None = None, request_id=None) -> Request:
        if request_id is None:
            request_id = self._next_id
            self._next_id += 1
        V = self.model.spec.vocab_size
        for t in prompt:
            if not 0 <= int(t) < V:
                raise ValueError(f"token id {t} is outside the vocabulary of {V}")
        return self.scheduler.add(request_id, prompt, params)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def abort(self, request_id) -> bool:
        return self.scheduler.abort(request_id)

    # ------------------------------------------------------------ one step
    def flush(self) -> list[Request]:
        """Read the tokens of the step in flight, if any.  Returns the requests that finished."""
        if self._in_flight is None:
            return []
        sched, handle = self._in_flight
        self._in_flight = None
        ids = self.sampler.collect(handle)
        rows = [s for s in sched if s.sample]
        return self.scheduler.resolve(sched, {s.request.request_id: t for s, t in zip(rows, ids)})

    def step(self) -> list[Request]:
        """Schedule, enqueue, draw, and read the tokens of the step BEFORE this one: the device is
        always one step ahead of what the host has seen.  Returns the requests that finished."""
        from .scheduler import PENDING
        sched = self.scheduler.schedule()
        finished = []
        if any(PENDING in s.tokens and len(s.tokens) > 1 for s in sched):
            # a re-admitted request would feed a token the host has not seen inside a portion
            finished += self.flush()
            sched = self.scheduler.schedule()
        if not sched:
            return finished + self.flush()
        entries = []
        for s in sched:
            r = s.request
            want = [len(s.tokens) - 1] if s.sample else []
            if s.tokens[-1] == PENDING:
                entries.append(StepEntry(r.request_id, [0], want, from_device=r.pending_row))
            else:
                entries.append(StepEntry(r.request_id, s.tokens, want))
        rows = [s for s in sched if s.sample]
        on_device = self.options.gpu_sampler and all(s.request.params.device_takes(self.model.spec.vocab_size) for s in rows)
        logits = self.runner.step(entries)
        if on_device:
            if any(PENDING in r.output and r.params.has_penalties and self._slot(r) is not None
                   and not self.sampler.holds_history(self._slot(r), r, len(r.output)) for r in (s.request for s in rows)):
                finished += self.flush()              # the history is counted anew from tokens the host knows
            inv_t = [0.0 if s.request.params.is_greedy else 1.0 / s.request.params.temperature for s in rows]
            us = [0.0 if s.request.params.is_greedy else s.request.rng.next_f32() for s in rows]
            if rows:
                requests = [s.request for s in rows]
                handle = self.sampler.sample_async(logits, inv_t, us, [r.params.device_filters for r in requests],
                                                   *self._histories_and_biases(requests))
            else:
                handle = (0, 0)
            self.scheduler.advance(sched)
            finished += self.flush()                  # the step before; this one is running meanwhile
            self._in_flight = (sched, handle) if rows else None
            return finished
        # Some request wants what the device sampler does not take (a top-k beyond 2048, a long
        # bias list): its logits go to the host sampler and nothing stays in flight.  Rows that the
        # device can draw are still drawn there (by the same kernel, from the same numbers of their
        # own generators), so a request's tokens do not depend on what its neighbours ask for.
        finished += self.flush()
        sampled = {}
        live = [i for i, s in enumerate(rows) if s.request.status != "finished"]   # (a stop token of the step before may just have ended one)
        on_dev = [i for i in live if self.options.gpu_sampler and rows[i].request.params.device_takes(self.model.spec.vocab_size)]
        if on_dev:
            params = [rows[i].request.params for i in on_dev]
            inv_t = [0.0 if p.is_greedy else 1.0 / p.temperature for p in params]
            us = [0.0 if p.is_greedy else rows[i].request.rng.next_f32() for i, p in zip(on_dev, params)]
            picked = logits if on_dev == list(range(logits.shape[0])) else self._pick_rows(logits, on_dev)
            for i, t in zip(on_dev, self.sampler.sample(picked, inv_t, us, [p.device_filters for p in params],
                                                        *self._histories_and_biases([rows[i].request for i in on_dev]))):
                sampled[rows[i].request.request_id] = t
        on_host = [i for i in live if i not in on_dev]
        if on_host:
            host = logits.to("cpu").numpy()
            for i in on_host:
                r = rows[i].request
                sampled[r.request_id] = sample_host(host[i], r.params, r.output, r.rng)
        return finished + self.scheduler.commit(sched, sampled)

    def _slot(self, request):
        held = self.runner.manager.live.get(request.request_id)
        return None if held is None else held.slot

    def _histories_and_biases(self, requests):
        """What the device sampler needs for penalties (the request's slot names its row of token
        counts) and bias, per row; ``None`` where nobody asks."""
        histories = biases = None
        if any(r.params.has_penalties for r in requests):
            # (a request that has just ended holds no slot any more; its row is drawn and dropped)
            histories = [(self._slot(r), r, r.output, *r.params.penalties)
                         if r.params.has_penalties and self._slot(r) is not None else None for r in requests]
        if any(r.params.logit_bias for r in requests):
            biases = [r.params.logit_bias for r in requests]
        return histories, biases

    def _pick_rows(self, logits, idx):
        """Rows ``idx`` of the step's logits, gathered on the device for the device sampler."""
        from ..kernels import ops
        n = len(idx)
        if self._pick_host is None:
            cap = max(self.options.inflight_slots, 1)
            self._pick_host = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._pick_dev = torch.empty(cap, dtype=torch.int32, device=self.model.rt.device)
        torch.cuda.current_stream().synchronize()          # the copy of the call before has left the pinned buffer
        self._pick_host[:n] = torch.tensor(idx, dtype=torch.int32)
        self._pick_dev[:n].copy_(self._pick_host[:n], non_blocking=True)
        out = self.model.rt.buffer("logits_for_device_sampler", n, logits.shape[1], torch.float32,
                                   max_rows=max(self.options.inflight_slots, 1))
        return ops.gather_rows(logits, self._pick_dev[:n], out)

    # ------------------------------------------------------------ whole generations
    def generate(self, prompts, params=None) -> list:
        """Generated token ids for each prompt (a list of token-id lists).  ``params`` is one
        ``SamplingParams`` for all or a list with one per prompt."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        reqs = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        while self.has_work():
            self.step()
        self.flush()
        return [list(r.output) for r in reqs]


def generate(model, prompts, max_new_tokens: int = 64, temperature: float = 0.0, seed: int = 0,
             dtype: str = "bfloat16", top_k=None, top_p=None, min_p=None, **engine_opts) -> list:
    """Generate from a model folder: token-id lists in, generated token-id lists out.

    ``engine_opts`` are fields of ``EngineOptions`` (``inflight_slots``, ``prefill_chunk_tokens``,
    ``paged_kv``, ``page_size``, ``ctx_cap``, ...).  Request ``i`` draws from a generator seeded
    with ``seed + i``."""
    opt = EngineOptions(dtype=dtype, seed=seed, **engine_opts)
    engine = LLMEngine.from_dir(model, opt)
    params = [SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, min_p=min_p,
                             max_tokens=max_new_tokens, seed=seed + i) for i in range(len(prompts))]
    return engine.generate(prompts, params)
