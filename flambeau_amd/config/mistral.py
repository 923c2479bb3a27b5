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
    eos_token_id: int | None = None      # the first end-of-sequence id (all of them: eos_token_ids)
    torch_dtype: str | None = None
    eos_token_ids: tuple = ()            # every id that ends a sequence
    layer_types: tuple | None = None     # per layer "sliding_attention" or "full_attention"; None: the window everywhere

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
        n_layers = r.integer("num_hidden_layers", minimum=1)
        _refuse_what_changes_the_arithmetic(raw, where)
        eos_ids = _int_tuple(raw.get("eos_token_id"), "eos_token_id", where)
        cfg = cls(
            hidden_size=hidden,
            num_hidden_layers=n_layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=r.integer("intermediate_size", minimum=1),
            vocab_size=r.integer("vocab_size", minimum=1),
            rms_norm_eps=r.number("rms_norm_eps", positive=True),
            rope_theta=_rope_theta(r, raw, where),
            max_position_embeddings=r.integer("max_position_embeddings", minimum=1),
            sliding_window=window,
            tie_word_embeddings=r.boolean("tie_word_embeddings", default=False),
            hidden_act=r.string("hidden_act", default="silu"),
            bos_token_id=r.integer("bos_token_id", default=None),
            eos_token_id=eos_ids[0] if eos_ids else None,
            torch_dtype=r.string("torch_dtype", default=None),
            eos_token_ids=eos_ids,
            layer_types=_layer_types(raw.get("layer_types"), n_layers, window, where),
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
        ids = d.pop("eos_token_ids")
        d["eos_token_id"] = list(ids) if len(ids) > 1 else (ids[0] if ids else None)
        d["layer_types"] = list(self.layer_types) if self.layer_types is not None else None
        return {k: v for k, v in d.items() if v is not None or k == "sliding_window"}

    def window_of_layer(self, layer: int) -> int:
        """Keys a query of this layer sees (0: all)."""
        if self.layer_types is None or self.layer_types[layer] == "sliding_attention":
            return self.sliding_window
        return 0


def _int_tuple(v, key, where) -> tuple:
    if v is None:
        return ()
    items = v if isinstance(v, list) else [v]
    for x in items:
        if isinstance(x, bool) or not isinstance(x, int):
            raise ConfigError(f"{where}: key '{key}' must be an integer or a list of them")
    return tuple(items)


_LAYER_TYPES = ("sliding_attention", "full_attention")


def _layer_types(v, n_layers, window, where):
    if v is None:
        return None
    if not isinstance(v, list) or len(v) != n_layers or any(t not in _LAYER_TYPES for t in v):
        raise ConfigError(f"{where}: key 'layer_types' must list one of {_LAYER_TYPES} for each of the {n_layers} layers")
    if "sliding_attention" in v and not window:
        raise ConfigError(f"{where}: 'layer_types' names sliding_attention but 'sliding_window' is not set")
    return tuple(v)


def _rope_theta(r: KeyReader, raw: dict, where: str) -> float:
    """``rope_theta``, or the same number inside ``rope_parameters`` (where newer files keep it).  Any
    scaling of the rotation (linear, dynamic, yarn, llama3, ...) changes the angles and is refused."""
    for key in ("rope_scaling", "rope_parameters"):
        v = raw.get(key)
        if v is None:
            continue
        if not isinstance(v, dict):
            raise ConfigError(f"{where}: key '{key}' must be an object")
        kind = v.get("rope_type", v.get("type", "default"))
        if kind != "default":
            raise ConfigError(f"{where}: key '{key}' asks for rotation scaling of type '{kind}', which this engine "
                              f"does not compute (only the unscaled rotation)")
        factor = v.get("factor")
        if factor is not None and float(factor) != 1.0:
            raise ConfigError(f"{where}: key '{key}' asks for a scaling factor of {factor}, which this engine does not compute")
    params = raw.get("rope_parameters")
    if isinstance(params, dict) and params.get("rope_theta") is not None:
        inner = KeyReader(params, f"{where}: rope_parameters").number("rope_theta", positive=True)
        outer = raw.get("rope_theta")
        if outer is not None and float(outer) != inner:
            raise ConfigError(f"{where}: 'rope_theta' {outer} and 'rope_parameters.rope_theta' {inner} differ")
        return inner
    return r.number("rope_theta", default=10000.0, positive=True)


def _refuse_what_changes_the_arithmetic(raw: dict, where: str) -> None:
    """Keys that switch on arithmetic this engine does not have must not be ignored: the model would
    load and give wrong logits."""
    for key in ("attention_bias", "mlp_bias"):
        v = raw.get(key)
        if v is not None and not isinstance(v, bool):
            raise ConfigError(f"{where}: key '{key}' must be true or false, got {v!r}")
        if v:
            raise ConfigError(f"{where}: key '{key}' is true; projections with a bias are not built")
