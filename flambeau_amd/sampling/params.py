"""Sampling options of a request, with the reference's names and meanings
(crates/runtime/src/sampling.rs:39-108; request defaults crates/server/src/state.rs:133-249)."""
from __future__ import annotations

from dataclasses import dataclass, field


@dataclass
class SamplingParams:
    temperature: float = 0.0            # <= 0: greedy argmax, first maximum wins
    top_k: int | None = None            # keep the k most probable
    top_p: float | None = None          # shortest prefix whose probability reaches p (0 < p < 1)
    min_p: float | None = None          # drop tokens below min_p * p_max
    repetition_penalty: float = 1.0     # seen tokens: l > 0 ? l / rp : l * rp
    presence_penalty: float = 0.0       # seen tokens: l -= pp
    frequency_penalty: float = 0.0      # seen tokens: l -= fp * count
    logit_bias: dict | None = None      # token id -> additive bias, after penalties
    seed: int | None = None             # xoshiro256** seed of this request
    max_tokens: int = 64                # generated tokens at most
    stop_token_ids: tuple = ()          # generation stops after one of these (besides eos)
    ignore_eos: bool = False

    def __post_init__(self):
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be at least 1")
        if self.top_k is not None and self.top_k < 1:
            raise ValueError("top_k must be at least 1")
        if self.repetition_penalty <= 0.0:
            raise ValueError("repetition_penalty must be positive")

    @property
    def is_greedy(self) -> bool:
        return self.temperature <= 0.0

    @property
    def has_penalties(self) -> bool:
        return (self.repetition_penalty != 1.0 or self.presence_penalty != 0.0
                or self.frequency_penalty != 0.0)

    @property
    def has_filters(self) -> bool:
        return self.top_k is not None or self.top_p is not None or self.min_p is not None

    @property
    def device_ok(self) -> bool:
        """Greedy and plain temperature sampling run on the device; penalties, bias and
        filters need the logits on the host."""
        return not (self.has_penalties or self.has_filters or self.logit_bias)
