"""Configuration and registry (no GPU)."""
import json

import pytest

from flambeau_amd.config import ConfigError, MistralConfig
from flambeau_amd.registry import (UnknownArchitecture, config_from_dict, config_from_dir, find_architecture,
                                   known_architectures)
from tiny_configs import TINY


def test_every_number_comes_from_the_file():
    for name, t in TINY.items():
        arch, cfg = config_from_dict(t["config"])
        raw = t["config"]
        assert arch.name == "MistralForCausalLM"
        assert cfg.hidden_size == raw["hidden_size"] and cfg.num_hidden_layers == raw["num_hidden_layers"]
        assert cfg.num_key_value_heads == raw["num_key_value_heads"]
        assert cfg.head_dim == raw.get("head_dim", raw["hidden_size"] // raw["num_attention_heads"])
        theta = raw["rope_theta"] if "rope_theta" in raw else raw["rope_parameters"]["rope_theta"]
        assert cfg.rms_norm_eps == raw["rms_norm_eps"] and cfg.rope_theta == theta
        assert cfg.sliding_window == (raw["sliding_window"] or 0)
        assert cfg.vocab_size == raw["vocab_size"] and cfg.tie_word_embeddings == raw["tie_word_embeddings"]
        spec = arch.build_spec(cfg)
        assert len(spec.layers) == raw["num_hidden_layers"] and len(spec.run_order) == raw["num_hidden_layers"]
        mixer = spec.layers[0].block.params["mixer"].params
        assert mixer["head_dim"] == cfg.head_dim and mixer["window"] == cfg.sliding_window
        types = raw.get("layer_types")
        for l, layer in enumerate(spec.layers):
            window = layer.block.params["mixer"].params["window"]
            assert window == (cfg.sliding_window if types is None or types[l] == "sliding_attention" else 0)
        assert mixer["position"].params["theta"] == cfg.rope_theta
        assert spec.layers[0].block.params["norm"].params["eps"] == cfg.rms_norm_eps


def test_defaults_of_the_format():
    raw = dict(TINY["A"]["config"])
    del raw["num_key_value_heads"], raw["rope_theta"], raw["sliding_window"], raw["tie_word_embeddings"]
    _, cfg = config_from_dict(raw)
    assert cfg.num_key_value_heads == cfg.num_attention_heads
    assert cfg.rope_theta == 10000.0 and cfg.sliding_window == 0 and cfg.tie_word_embeddings is False
    assert cfg.head_dim == 16


def test_round_trip_through_to_dict():
    for t in TINY.values():
        _, cfg = config_from_dict(t["config"])
        _, again = config_from_dict(cfg.to_dict())
        assert again == cfg


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads", "intermediate_size",
                                 "vocab_size", "rms_norm_eps", "max_position_embeddings"])
def test_missing_key_is_named(key):
    raw = dict(TINY["B"]["config"])
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(raw)


def test_bad_values_are_refused():
    base = TINY["A"]["config"]
    for patch, pattern in [
        ({"num_key_value_heads": 3}, "not a multiple"),
        ({"head_dim": 15}, "even"),
        ({"hidden_act": "gelu"}, "hidden_act"),
        ({"hidden_size": "64"}, "integer"),
        ({"rms_norm_eps": 0}, "> 0"),
        ({"num_attention_heads": 5}, "head_dim"),
        ({"tie_word_embeddings": "no"}, "true or false"),
    ]:
        raw = dict(base)
        raw.update(patch)
        with pytest.raises(ConfigError, match=pattern):
            config_from_dict(raw)


def test_keys_that_change_the_arithmetic_are_read_or_refused():
    base = TINY["A"]["config"]
    for patch, pattern in [
        ({"rope_scaling": {"rope_type": "linear", "factor": 2.0}}, "rotation scaling of type 'linear'"),
        ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "yarn"),
        ({"rope_parameters": {"rope_type": "llama3", "rope_theta": 1e4}}, "llama3"),
        ({"rope_scaling": {"rope_type": "default", "factor": 8.0}}, "factor"),
        ({"rope_scaling": "linear"}, "must be an object"),
        ({"rope_parameters": {"rope_type": "default", "rope_theta": 5e5}}, "differ"),      # base says 1e4
        ({"attention_bias": True}, "attention_bias"),
        ({"mlp_bias": True}, "mlp_bias"),
        ({"mlp_bias": "yes"}, "true or false"),
        ({"layer_types": ["sliding_attention"]}, "layer_types"),
        ({"layer_types": ["sliding_attention", "chunked"]}, "layer_types"),
        ({"sliding_window": None, "layer_types": ["sliding_attention", "full_attention"]}, "sliding_window"),
        ({"eos_token_id": [2, "x"]}, "eos_token_id"),
    ]:
        raw = dict(base)
        raw.update(patch)
        with pytest.raises(ConfigError, match=pattern):
            config_from_dict(raw)
    # the harmless forms are read
    raw = dict(base, rope_scaling=None, attention_bias=False, mlp_bias=False, eos_token_id=[2, 9, 5])
    del raw["rope_theta"]
    raw["rope_parameters"] = {"rope_type": "default", "rope_theta": 7.5e5}
    _, cfg = config_from_dict(raw)
    assert cfg.rope_theta == 7.5e5 and cfg.eos_token_ids == (2, 9, 5) and cfg.eos_token_id == 2
    arch, _ = config_from_dict(raw)
    assert arch.build_spec(cfg).eos_token_ids == (2, 9, 5)
    _, cfg = config_from_dict(dict(base, eos_token_id=3))
    assert cfg.eos_token_ids == (3,)
    _, cfg = config_from_dict(TINY["D"]["config"])
    assert [cfg.window_of_layer(l) for l in range(4)] == [20, 0, 0, 20]


def test_unknown_architecture_lists_the_known_ones():
    raw = dict(TINY["A"]["config"], architectures=["LlamaForCausalLM"])
    with pytest.raises(UnknownArchitecture, match="MistralForCausalLM"):
        config_from_dict(raw)
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in raw.items() if k != "architectures"})
    assert "MistralForCausalLM" in known_architectures()
    assert find_architecture("MistralForCausalLM").config_class is MistralConfig


def test_config_from_dir(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY["C"]["config"]))
    _, cfg = config_from_dir(tmp_path)
    assert cfg.tie_word_embeddings and cfg.sliding_window == 24
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        config_from_dir(tmp_path)
    with pytest.raises(ConfigError, match="no such file"):
        config_from_dir(tmp_path / "nowhere")


def test_sizes_no_kernel_takes_are_refused_when_the_model_is_built():
    """A head size beyond the attention kernels' limit passes the configuration (it is a kernel's limit,
    not the architecture's) and is refused when the model's parts are made, before any weight is read
    or any step runs, with an error that names the key."""
    from flambeau_amd.kernels import ops
    from flambeau_amd.models.mistral import mistral_spec
    from flambeau_amd.parts import BLOCKS
    limit = ops.attention_max_head_dim()
    assert limit >= 256
    raw = dict(architectures=["MistralForCausalLM"], hidden_size=64, num_hidden_layers=1, num_attention_heads=2,
               num_key_value_heads=1, intermediate_size=96, vocab_size=50, rms_norm_eps=1e-5, max_position_embeddings=64)
    ok = mistral_spec(MistralConfig.from_dict(dict(raw, head_dim=limit), "config"))
    BLOCKS.create(ok.layers[0].block)
    spec = mistral_spec(MistralConfig.from_dict(dict(raw, head_dim=limit + 16), "config"))
    with pytest.raises(ConfigError, match="'head_dim'"):
        BLOCKS.create(spec.layers[0].block)
