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
                                   max_queue_depth=opt.max_queue_depth, eos_token_id=spec.eos_token_id,
                                   default_seed=opt.seed)
        self.sampler = DeviceSampler(model.rt.device, max(opt.inflight_slots, 1))
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
    def step(self) -> list[Request]:
        """Schedule, run, sample, commit.  Returns the requests that finished in this step."""
        sched = self.scheduler.schedule()
        if not sched:
            return []
        entries = [StepEntry(s.request.request_id, s.tokens, [len(s.tokens) - 1] if s.sample else [])
                   for s in sched]
        logits = self.runner.step(entries)
        sampled = {}
        rows = [s for s in sched if s.sample]
        if rows:
            on_device = self.options.gpu_sampler and all(s.request.params.device_ok for s in rows)
            if on_device:
                inv_t = [0.0 if s.request.params.is_greedy else 1.0 / s.request.params.temperature for s in rows]
                us = [0.0 if s.request.params.is_greedy else s.request.rng.next_f32() for s in rows]
                ids = self.sampler.sample(logits, inv_t, us)
            else:
                host = logits.to("cpu").numpy()
                ids = [sample_host(host[i], s.request.params, s.request.output, s.request.rng)
                       for i, s in enumerate(rows)]
            for s, tok in zip(rows, ids):
                sampled[s.request.request_id] = tok
        return self.scheduler.commit(sched, sampled)

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
