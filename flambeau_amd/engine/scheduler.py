"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.  Host logic only; it talks to the ``CacheManager`` and never to the GPU.

One loop, no thread per request: ``schedule()`` picks this step's entries, the step function
runs them, ``commit()`` takes the sampled tokens.  Rules:

* Every running request whose known tokens are all in the cache but the last one contributes
  that one token (a decode row).  Decode rows are scheduled before prompt tokens.
* What is left of ``max_batch_tokens`` is dealt to requests that still have prompt (or, after
  a pre-emption, earlier output) to run, in order of arrival, each getting at most
  ``prefill_chunk_tokens`` per step; several portions may share a step.  With a ``row_granule``
  the portions' share is rounded down so that the step's rows are a multiple of it (the matrix
  kernels work on tiles of rows; 8 decode rows beside a portion of 504 cost less than beside 512).
* A waiting request is admitted when a slot is free and the free pages cover its first portion.
  Order of arrival is kept: nobody overtakes the head of the queue.
* Pages are asked for before the batch is built, so the step itself never runs out.  If a decode
  row cannot get its page, the running request that was admitted last is pre-empted: its pages
  and slot are given back and it returns to the head of the queue with everything it has
  produced so far as its prompt (recomputed when it resumes).  A request that could never fit
  in the pool is refused when it is added; so is any request while the queue is full.

The reference schedules inside its HTTP server: admission against ``inflight_slots +
max_queue_depth`` (crates/server/src/routes.rs:472-496), prompts cut into
``prefill_chunk_tokens`` portions with at most one portion per forward
(crates/server/src/routes/decode_loop.rs:371,418-474), decode rows drained from a pending queue
(routes.rs:631-733); when pages run out the forward errors and the request dies
(crates/forward/src/core/composites/standard_attn.rs:449-458).
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams
from ..sampling.rng import Xoshiro256


class AdmissionError(RuntimeError):
    """A request that is refused when it is added."""


PENDING = -1     # a token that was drawn on the device and that the host has not seen yet


@dataclass
class Request:
    request_id: object
    prompt: list
    params: SamplingParams
    output: list = field(default_factory=list)
    n_computed: int = 0                 # tokens whose keys are in the cache
    status: str = "waiting"             # waiting, running, finished
    finish_reason: str | None = None    # "stop", "length"
    n_preempted: int = 0
    rng: Xoshiro256 | None = None
    arrival: int = 0
    pending_row: int | None = None      # where the PENDING token lies in the sampler's output buffer
    reported: bool = False

    @property
    def tokens(self) -> list:
        return self.prompt + self.output

    def token_at(self, i: int):
        """Token ``i`` of prompt + output, without joining the two lists."""
        n = len(self.prompt)
        return self.prompt[i] if i < n else self.output[i - n]

    def token_slice(self, a: int, b: int) -> list:
        """Tokens ``[a, b)`` of prompt + output; copies only what it returns."""
        n = len(self.prompt)
        if b <= n:
            return self.prompt[a:b]
        if a >= n:
            return self.output[a - n:b - n]
        return self.prompt[a:] + self.output[:b - n]

    @property
    def n_pending(self) -> int:
        return len(self.prompt) + len(self.output) - self.n_computed


@dataclass
class Scheduled:
    request: Request
    tokens: list
    sample: bool                        # the portion reaches the last known token: sample after it


class Scheduler:
    def __init__(self, manager: CacheManager, *, max_batch_tokens: int, prefill_chunk_tokens: int = 512,
                 max_queue_depth: int = 0, eos_token_id=None, default_seed: int = 0, row_granule: int = 1):
        if max_batch_tokens < 1 or prefill_chunk_tokens < 1:
            raise ValueError("token budgets must be positive")
        self.manager = manager
        self.max_batch_tokens = max_batch_tokens
        self.prefill_chunk_tokens = prefill_chunk_tokens
        # The kernels work on tiles of this many rows: a step of 520 rows costs what 640 cost.  Where a
        # step holds more rows than one tile, the prompt portions are cut so that decode rows and
        # portions together fill whole tiles.
        self.row_granule = max(1, int(row_granule))
        self.max_queue_depth = max_queue_depth      # 0: no limit (routes.rs:481 "0 disables")
        # one id or several: any of them ends a request
        if eos_token_id is None:
            self.eos_token_ids = frozenset()
        elif isinstance(eos_token_id, int):
            self.eos_token_ids = frozenset([eos_token_id])
        else:
            self.eos_token_ids = frozenset(int(t) for t in eos_token_id)
        self.default_seed = default_seed
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []            # in order of admission
        self._arrivals = 0
        self.n_preemptions = 0

    # ------------------------------------------------------------ adding
    def _peak_pages(self, n_tokens: int) -> list[int]:
        """Most pages per group a request of ``n_tokens`` holds at any time."""
        ps = self.manager.page_size
        out = []
        for g in self.manager.groups:
            full = -(-n_tokens // ps)
            if g.window > 0:
                # live keys: a window behind the newest portion, plus page rounding at both ends
                span = g.window + min(self.prefill_chunk_tokens, self.max_batch_tokens)
                full = min(full, -(-span // ps) + 1)
            out.append(full)
        return out

    def add(self, request_id, prompt, params: SamplingParams | None = None) -> Request:
        params = params or SamplingParams()
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise AdmissionError(f"request {request_id!r}: empty prompt")
        if any(r.request_id == request_id for r in list(self.waiting) + self.running):
            raise AdmissionError(f"request {request_id!r} is already known")
        if self.max_queue_depth and len(self.waiting) >= self.max_queue_depth:
            raise AdmissionError(f"request {request_id!r}: queue full ({self.max_queue_depth} waiting)")
        if len(prompt) + 1 > self.manager.max_seq_len:
            raise AdmissionError(
                f"request {request_id!r}: a prompt of {len(prompt)} tokens leaves no room under the "
                f"maximum length {self.manager.max_seq_len}")
        # the last token drawn is never fed, so the cache holds at most this many tokens
        total = min(len(prompt) + params.max_tokens - 1, self.manager.max_seq_len)
        for g, (need, pool) in enumerate(zip(self._peak_pages(total), self.manager.pools)):
            if need > pool.n_pages:
                raise AdmissionError(
                    f"request {request_id!r}: needs {need} pages in cache group {g}, the pool has {pool.n_pages}")
        seed = params.seed if params.seed is not None else self.default_seed + self._arrivals
        req = Request(request_id, prompt, params, rng=Xoshiro256(seed), arrival=self._arrivals)
        self._arrivals += 1
        self.waiting.append(req)
        return req

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def abort(self, request_id) -> bool:
        """Drop a request wherever it is; its pages and slot are given back."""
        for r in list(self.waiting):
            if r.request_id == request_id:
                self.waiting.remove(r)
                r.status, r.finish_reason = "finished", "abort"
                return True
        for r in self.running:
            if r.request_id == request_id:
                self.running.remove(r)
                self.manager.release(request_id)
                r.status, r.finish_reason = "finished", "abort"
                return True
        return False

    # ------------------------------------------------------------ scheduling
    def _free_after(self, planned) -> list[int]:
        """Free pages per group once the planned entries have taken theirs."""
        free = self.manager.free_pages()
        for req, upto in planned:
            for g, k in enumerate(self.manager.pages_needed(req.request_id, upto)):
                free[g] -= k
        return free

    def _fits(self, planned, req, upto) -> bool:
        free = self._free_after(planned)
        return all(k <= f for k, f in zip(self.manager.pages_needed(req.request_id, upto), free))

    def _preempt(self, req: Request) -> None:
        self.manager.release(req.request_id)
        self.running.remove(req)
        req.status = "waiting"
        req.n_computed = 0
        req.n_preempted += 1
        self.n_preemptions += 1
        self.waiting.appendleft(req)

    def schedule(self) -> list[Scheduled]:
        budget = self.max_batch_tokens
        out: list[Scheduled] = []
        planned: list = []          # (request, tokens in cache after this step)

        # 1. decode rows, oldest first; pre-empt the newest when a page is missing
        decoders = [r for r in self.running if r.n_pending == 1]
        i = 0
        while i < len(decoders) and budget > 0:
            r = decoders[i]
            if r not in self.running:       # pre-empted below
                i += 1
                continue
            upto = r.n_computed + 1
            if self._fits(planned, r, upto):
                out.append(Scheduled(r, [r.token_at(r.n_computed)], True))
                planned.append((r, upto))
                budget -= 1
                i += 1
                continue
            victim = self.running[-1]
            if any(s.request is victim for s in out):
                # the newest is already in this step: take it out again, then give up its pages
                out = [s for s in out if s.request is not victim]
                planned = [p for p in planned if p[0] is not victim]
                budget += 1
            self._preempt(victim)
            # r itself may have been the victim; the loop looks at r again otherwise

        # 2. portions of running requests, in order of admission; their budget is rounded down so that
        # the step's rows fill whole tiles (never below half the budget)
        g = self.row_granule
        if g > 1 and budget > 0:
            used = self.max_batch_tokens - budget
            whole = (used + budget) // g * g - used
            if whole >= max(1, budget // 2):
                budget = whole
        for r in list(self.running):
            if budget <= 0:
                break
            if r.n_pending <= 1:
                continue
            k = self._portion(planned, r, min(r.n_pending, budget, self.prefill_chunk_tokens))
            if k <= 0:
                continue
            out.append(Scheduled(r, r.token_slice(r.n_computed, r.n_computed + k), k == r.n_pending))
            planned.append((r, r.n_computed + k))
            budget -= k

        # 3. admit from the queue, head first
        while self.waiting and budget > 0 and self.manager.n_free_slots > 0:
            r = self.waiting[0]
            self.manager.admit(r.request_id)
            k = self._portion(planned, r, min(r.n_pending, budget, self.prefill_chunk_tokens))
            if k <= 0:
                self.manager.release(r.request_id)
                break
            self.waiting.popleft()
            r.status = "running"
            self.running.append(r)
            out.append(Scheduled(r, r.token_slice(0, k), k == r.n_pending))
            planned.append((r, k))
            budget -= k

        # 4. nothing can move although requests are running: free the newest one's pages
        if not out and self.running:
            self._preempt(self.running[-1])
            return self.schedule()
        return out

    def _portion(self, planned, req, k: int) -> int:
        """The longest portion <= k whose pages are free (whole pages count)."""
        if k <= 0:
            return 0
        if self._fits(planned, req, req.n_computed + k):
            return k
        free = self._free_after(planned)
        ps = self.manager.page_size
        held = [len(t) for t in self.manager.live[req.request_id].tables]
        room = min((h + f) * ps for h, f in zip(held, free)) - req.n_computed if held else k
        return max(0, min(k, room))

    # ------------------------------------------------------------ after the step
    def commit(self, scheduled: list, sampled: dict) -> list[Request]:
        """``sampled``: request id -> token drawn after its portion (for entries with
        ``sample``).  Returns the requests that finished; their pages and slots are free."""
        self.advance(scheduled)
        return self.resolve(scheduled, sampled)

    # The commit in two halves, for an engine that enqueues the next step before it has seen the
    # tokens of this one: ``advance`` right after the step is enqueued (what does not depend on
    # the tokens' values), ``resolve`` when the values have arrived.
    def advance(self, scheduled: list) -> None:
        row = -1
        for s in scheduled:
            r = s.request
            if s.sample:
                row += 1
            if r.status == "finished":
                continue                         # a stop token ended it while this step was enqueued
            r.n_computed += len(s.tokens)
            if not s.sample:
                continue
            r.output.append(PENDING)
            r.pending_row = row
            if len(r.output) >= r.params.max_tokens or len(r.prompt) + len(r.output) >= self.manager.max_seq_len:
                # the length ends it whatever the token is; pages are free for steps enqueued later
                r.finish_reason = "length"
                r.status = "finished"
                self.running.remove(r)
                self.manager.release(r.request_id)

    def resolve(self, scheduled: list, sampled: dict) -> list[Request]:
        """Fill in the drawn tokens; a stop token ends its request (a step that was enqueued for it
        meanwhile is wasted: its token is dropped)."""
        finished = []
        for s in scheduled:
            if not s.sample:
                continue
            r = s.request
            if PENDING not in r.output:
                continue                         # stopped earlier: this was a step beyond its end
            at = r.output.index(PENDING)
            tok = int(sampled[r.request_id])
            r.output[at] = tok
            if r.pending_row is not None and PENDING not in r.output:
                r.pending_row = None
            stop = (not r.params.ignore_eos and tok in self.eos_token_ids) or tok in r.params.stop_token_ids
            if stop:
                del r.output[at + 1:]
                r.pending_row = None
                r.finish_reason = "stop"
                if r.status != "finished":
                    r.status = "finished"
                    if r in self.running:
                        self.running.remove(r)
                        self.manager.release(r.request_id)
                    elif r in self.waiting:
                        self.waiting.remove(r)
            if r.status == "finished" and PENDING not in r.output and not r.reported:
                r.reported = True
                finished.append(r)
        return finished
