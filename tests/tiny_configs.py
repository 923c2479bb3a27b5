"""Tiny configurations of the architecture for the tests.  They differ in every size and
option: layers, width, head counts and groups (GQA, MQA, MHA), head size (derived, explicit
and not width/heads), intermediate size, vocabulary (none a power of two but A's), theta,
window (16, none, 24 = no multiple of a page; D: a window in two of its four layers only, so its
cache has two groups of layers with pages of their own), eps, tied or untied head, weight scale,
one or several end-of-sequence ids."""
import torch

from flambeau_amd.weights import write_random_model


def _cfg(**kw):
    base = {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_act": "silu"}
    base.update(kw)
    return base


TINY = {
    "A": dict(
        config=_cfg(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
                    intermediate_size=160, vocab_size=256, rope_theta=10000.0, sliding_window=16,
                    rms_norm_eps=1e-5, max_position_embeddings=128, tie_word_embeddings=False),
        seed=0, std=0.02, gain_std=0.01, page_size=8),
    "B": dict(
        config=_cfg(num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=1,
                    head_dim=24, intermediate_size=224, vocab_size=384, rope_theta=1e6,
                    sliding_window=None, rms_norm_eps=1e-6, max_position_embeddings=256,
                    tie_word_embeddings=False),
        seed=2, std=0.05, gain_std=0.01, page_size=16),
    "C": dict(
        config=_cfg(num_hidden_layers=2, hidden_size=80, num_attention_heads=5, num_key_value_heads=5,
                    head_dim=32, intermediate_size=136, vocab_size=300, rope_theta=5e5,
                    sliding_window=24, rms_norm_eps=1e-4, max_position_embeddings=640,
                    tie_word_embeddings=True),
        seed=5, std=0.04, gain_std=0.02, page_size=16),
    "D": dict(
        config=_cfg(num_hidden_layers=4, hidden_size=48, num_attention_heads=3, num_key_value_heads=1,
                    head_dim=16, intermediate_size=72, vocab_size=210, rope_parameters={"rope_type": "default", "rope_theta": 2.5e4},
                    sliding_window=20, layer_types=["sliding_attention", "full_attention", "full_attention", "sliding_attention"],
                    rms_norm_eps=3e-6, max_position_embeddings=512, tie_word_embeddings=False,
                    eos_token_id=[7, 11]),
        seed=9, std=0.06, gain_std=0.03, page_size=8),
}

STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def write_tiny(name, out_dir, store="float32"):
    t = TINY[name]
    return write_random_model(t["config"], out_dir, seed=t["seed"], std=t["std"], gain_std=t["gain_std"],
                              store_dtype=STORE[store])


def write_sharpened(name, out_dir, store="float32", factor=12.0):
    """The tiny model with its query and key matrices scaled up, so that attention is peaked:
    single keys (far ones, those at a window's edge, those at a page's edge) carry visible
    weight and a fault in any one of them shows in the logits."""
    from flambeau_amd.weights import SafetensorsFile, write_safetensors
    d = write_tiny(name, out_dir, store)
    f = SafetensorsFile(d / "model.safetensors")
    tensors = {}
    for n in f.names():
        t = f.read(n)
        if n.endswith("q_proj.weight") or n.endswith("k_proj.weight"):
            t = (t.float() * factor).to(t.dtype)
        tensors[n] = t
    f.close()
    write_safetensors(d / "model.safetensors", tensors)
    return d
