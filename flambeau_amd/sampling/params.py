"""Sampling options of a request, with the reference's names and meanings
(crates/runtime/src/sampling.rs:39-108; request defaults crates/server/src/state.rs:133-249)."""
from __future__ import annotations

from dataclasses import dataclass, field

DEVICE_TOP_K_MAX = 2048       # candidates the device sampler keeps (fl_sample_filtered_max_k)
DEVICE_BIAS_MAX = 256         # logit-bias entries of one request that the device sampler takes
DEVICE_FILTER_VOCAB_MAX = 261120     # the largest vocabulary the filtered draw takes (fl_sample_filtered_max_vocab)


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
        """Penalties, a bias of up to 256 entries, greedy sampling, the temperature draw and the filters
        (top-k up to 2048, top-p, min-p) run on the device; what is beyond goes to the host sampler."""
        return not ((self.logit_bias is not None and len(self.logit_bias) > DEVICE_BIAS_MAX)
                    or (self.top_k is not None and self.top_k > DEVICE_TOP_K_MAX))

    def device_takes(self, vocab_size: int) -> bool:
        """``device_ok`` for a model's vocabulary: the filtered draw keeps a count per 1,024 tokens in a
        byte, so filters over a vocabulary beyond 261,120 go to the host sampler too."""
        if self.has_filters and not self.is_greedy and vocab_size > DEVICE_FILTER_VOCAB_MAX:
            return False
        return self.device_ok

    @property
    def penalties(self) -> tuple:
        return (self.repetition_penalty, self.presence_penalty, self.frequency_penalty)

    @property
    def device_filters(self) -> tuple:
        """``(top_k, top_p, min_p)`` as the device sampler takes them: 0 for what is not asked for."""
        top_p = self.top_p if self.top_p is not None and 0.0 < self.top_p < 1.0 else 0.0
        min_p = self.min_p if self.min_p is not None and self.min_p > 0.0 else 0.0
        top_k = int(self.top_k) if self.top_k is not None else (DEVICE_TOP_K_MAX if (top_p or min_p) else 0)
        if self.has_filters and not (top_k or top_p or min_p):
            top_k = DEVICE_TOP_K_MAX          # filters that cut nothing (top_p = 1) still draw among the 2048 most probable
        return (top_k, top_p, min_p)
