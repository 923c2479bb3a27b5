"""MistralConfig: the numbers of a Mistral dense decoder, read from config.json.

Counterpart of the reference's typed per-architecture config
(crates/models/qwen35-v2/src/config.rs:6-109), for the Hugging Face keys of
``MistralForCausalLM`` instead of GGUF metadata.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class MistralConfig:
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    sliding_window: int          # keys a query sees, itself included; 0 = all
    tie_word_embeddings: bool
    hidden_act: str
    bos_token_id: int | None = None
    eos_token_id: int | None = None
    torch_dtype: str | None = None

    architecture = "MistralForCausalLM"

    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "MistralConfig":
        r = KeyReader(raw, where)
        hidden = r.integer("hidden_size", minimum=1)
        heads = r.integer("num_attention_heads", minimum=1)
        kv_heads = r.integer("num_key_value_heads", default=heads, minimum=1)
        head_dim = r.integer("head_dim", default=None, minimum=1)
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(
                    f"{where}: 'hidden_size' {hidden} is not a multiple of 'num_attention_heads' "
                    f"{heads} and no 'head_dim' is given")
            head_dim = hidden // heads
        window = r.integer("sliding_window", default=0, minimum=0)
        cfg = cls(
            hidden_size=hidden,
            num_hidden_layers=r.integer("num_hidden_layers", minimum=1),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=r.integer("intermediate_size", minimum=1),
            vocab_size=r.integer("vocab_size", minimum=1),
            rms_norm_eps=r.number("rms_norm_eps", positive=True),
            rope_theta=r.number("rope_theta", default=10000.0, positive=True),
            max_position_embeddings=r.integer("max_position_embeddings", minimum=1),
            sliding_window=window,
            tie_word_embeddings=r.boolean("tie_word_embeddings", default=False),
            hidden_act=r.string("hidden_act", default="silu"),
            bos_token_id=r.integer("bos_token_id", default=None),
            eos_token_id=_first_int(raw.get("eos_token_id"), where),
            torch_dtype=r.string("torch_dtype", default=None),
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"{where}: 'num_attention_heads' {self.num_attention_heads} is not a multiple of "
                f"'num_key_value_heads' {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"{where}: 'head_dim' {self.head_dim} must be even (rotation pairs)")
        if self.hidden_act != "silu":
            raise ConfigError(f"{where}: 'hidden_act' must be 'silu', got '{self.hidden_act}'")

    def to_dict(self) -> dict:
        """A config.json dictionary that ``from_dict`` reads back to this config."""
        d = asdict(self)
        d["architectures"] = [self.architecture]
        d["model_type"] = "mistral"
        d["sliding_window"] = self.sliding_window or None
        return {k: v for k, v in d.items() if v is not None or k == "sliding_window"}


def _first_int(v, where):
    if v is None:
        return None
    if isinstance(v, list):
        v = v[0] if v else None
        if v is None:
            return None
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"{where}: key 'eos_token_id' must be an integer or a list of them")
    return v
