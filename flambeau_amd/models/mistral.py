"""Mistral dense (``MistralForCausalLM``) as a description of parts.

Pre-norm decoder: grouped-query attention with split-half rotation and an optional sliding
window, RMSNorm, SwiGLU, untied (or tied) output head.  The reference names the architecture
in scope (README.md:20) and runs it, in its own terms, as the loop of
crates/forward/README.md:22-41 with attn_q_gated=false, no q/k norms, rotated_dims=head_dim
and Activation::SwiGLU (crates/forward/tests/synth_dense.rs:58-108).  Tensor names are those of
Hugging Face checkpoints of this architecture.
"""
from __future__ import annotations

from ..config.mistral import MistralConfig
from ..parts import PartSpec
from ..registry import register_architecture
from .decoder import LayerSpec, ModelSpec, RunEntry


def mistral_spec(cfg: MistralConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", dict(hidden_size=cfg.hidden_size, eps=cfg.rms_norm_eps))
    position = PartSpec("rope_neox", dict(head_dim=cfg.head_dim, theta=cfg.rope_theta))
    ffn = PartSpec("swiglu", dict(hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size))

    def block(window):
        mixer = PartSpec("paged_gqa_attention", dict(
            hidden_size=cfg.hidden_size, n_heads=cfg.num_attention_heads,
            n_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim,
            window=window, position=position))
        return PartSpec("prenorm", dict(mixer=mixer, feed_forward=ffn, norm=norm))

    layers = []
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        layers.append(LayerSpec(block(cfg.window_of_layer(l)), {
            "mixer_norm.weight": p + "input_layernorm.weight",
            "mixer.q.weight": p + "self_attn.q_proj.weight",
            "mixer.k.weight": p + "self_attn.k_proj.weight",
            "mixer.v.weight": p + "self_attn.v_proj.weight",
            "mixer.o.weight": p + "self_attn.o_proj.weight",
            "ffn_norm.weight": p + "post_attention_layernorm.weight",
            "ffn.gate.weight": p + "mlp.gate_proj.weight",
            "ffn.up.weight": p + "mlp.up_proj.weight",
            "ffn.down.weight": p + "mlp.down_proj.weight",
        }))
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        layers=layers,
        run_order=[RunEntry(l) for l in range(cfg.num_hidden_layers)],
        final_norm=norm,
        names={"embedding.weight": "model.embed_tokens.weight",
               "final_norm.weight": "model.norm.weight",
               "head.weight": "lm_head.weight"},
        tied_head=cfg.tie_word_embeddings,
        eos_token_id=cfg.eos_token_id,
        bos_token_id=cfg.bos_token_id,
        eos_token_ids=cfg.eos_token_ids,
        # tensors that files of this architecture may hold and the model does not read
        ignored_tensors=("*.rotary_emb.inv_freq",) + (("lm_head.weight",) if cfg.tie_word_embeddings else ()),
    )


register_architecture("MistralForCausalLM", MistralConfig, mistral_spec)
