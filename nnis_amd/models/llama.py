"""Llama as a model description: pre-norm blocks of grouped-query attention
with rotate-half RoPE and a SiLU-gated feed-forward, RMSNorm, tied or untied
head.  Formulas and their order:
/root/reference/crates/nnis-model/src/runtime.rs:918-1120; tensor names:
/root/reference/crates/nnis-model/src/safetensors_loader.rs:440-551.
"""

from __future__ import annotations

from ..config.llama import LlamaConfig
from .spec import ModelSpec, ScheduleEntry


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    layers = []
    for index in range(cfg.num_hidden_layers):
        prefix = f"model.layers.{index}."
        layers.append(
            {
                "kind": "pre_norm",
                "width": cfg.hidden_size,
                "norm1": {
                    "kind": "rms",
                    "width": cfg.hidden_size,
                    "eps": cfg.rms_norm_eps,
                    "weight": prefix + "input_layernorm.weight",
                },
                "mixer": {
                    "kind": "causal_attention",
                    "width": cfg.hidden_size,
                    "heads": cfg.num_attention_heads,
                    "kv_heads": cfg.num_key_value_heads,
                    "head_dim": cfg.head_dim,
                    "position": "rope",
                    "q": prefix + "self_attn.q_proj.weight",
                    "k": prefix + "self_attn.k_proj.weight",
                    "v": prefix + "self_attn.v_proj.weight",
                    "o": prefix + "self_attn.o_proj.weight",
                },
                "norm2": {
                    "kind": "rms",
                    "width": cfg.hidden_size,
                    "eps": cfg.rms_norm_eps,
                    "weight": prefix + "post_attention_layernorm.weight",
                },
                "feed_forward": {
                    "kind": "gated",
                    "width": cfg.hidden_size,
                    "inner": cfg.intermediate_size,
                    "activation": cfg.hidden_act,
                    "gate": prefix + "mlp.gate_proj.weight",
                    "up": prefix + "mlp.up_proj.weight",
                    "down": prefix + "mlp.down_proj.weight",
                },
            }
        )
    spec = ModelSpec(
        architecture=cfg.architecture,
        width=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings,
        stored_dtype=cfg.torch_dtype,
        embedding={
            "kind": "table",
            "vocab_size": cfg.vocab_size,
            "width": cfg.hidden_size,
            "weight": "model.embed_tokens.weight",
        },
        positions={
            "rope": {
                "kind": "rotary_half",
                "rot_dim": cfg.head_dim,
                "theta": cfg.rope_theta,
                "max_positions": cfg.max_position_embeddings,
            }
        },
        layers=layers,
        schedule=[ScheduleEntry(layer=i) for i in range(cfg.num_hidden_layers)],
        final_norm={
            "kind": "rms",
            "width": cfg.hidden_size,
            "eps": cfg.rms_norm_eps,
            "weight": "model.norm.weight",
        },
        head={
            "kind": "linear",
            "vocab_size": cfg.vocab_size,
            "width": cfg.hidden_size,
            "weight": "lm_head.weight",
            # safetensors_loader.rs:755-786: lm_head.weight wins when present,
            # else the embedding stands in if the configuration ties them
            "tied_to": "model.embed_tokens.weight" if cfg.tie_word_embeddings else None,
        },
        stop_token_ids=cfg.eos_token_ids,
        # a buffer that older Llama checkpoints carry beside the weights (the tables are made from theta here)
        ignored_tensor_suffixes=("rotary_emb.inv_freq",),
        config_json=cfg.to_dict(),
    )
    spec.validate()
    return spec
