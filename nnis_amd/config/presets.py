"""Named configurations: the model shapes this library is measured on and the
two tiny ones its smoke runs use, as the config.json each would carry.

SmolLM2-135M and TinyLlama-1.1B are the reference's pinned checkpoints
(/root/reference/crates/nnis-model/src/exact_checkpoint_spec.rs:219-259);
SmolLM2-1.7B has the same architecture at 24 layers of width 2048; "llama-8b"
is a fourth shape for measurements only.  A preset
gives sizes only: weights come from a checkpoint of that shape or from the
random-weights mode (``write_random_model(folder, preset("smollm2-135m"),
seed)``).
"""

from __future__ import annotations

from typing import Any, Dict, List

from ..errors import InvalidInput


def _llama(**sizes) -> Dict[str, Any]:
    config = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu", "torch_dtype": "bfloat16"}
    config.update(sizes)
    return config


_PRESETS: Dict[str, Dict[str, Any]] = {
    "smollm2-135m": _llama(
        num_hidden_layers=30, hidden_size=576, num_attention_heads=9, num_key_value_heads=3, head_dim=64,
        intermediate_size=1536, vocab_size=49152, rope_theta=100000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
        max_position_embeddings=8192, eos_token_id=0),
    "smollm2-1.7b": _llama(
        num_hidden_layers=24, hidden_size=2048, num_attention_heads=32, num_key_value_heads=32, head_dim=64,
        intermediate_size=8192, vocab_size=49152, rope_theta=130000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
        max_position_embeddings=8192, eos_token_id=0),
    "tinyllama-1.1b": _llama(
        num_hidden_layers=22, hidden_size=2048, num_attention_heads=32, num_key_value_heads=4, head_dim=64,
        intermediate_size=5632, vocab_size=32000, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
        max_position_embeddings=2048, eos_token_id=2),
    # beyond the reference's checkpoints: the sizes of an 8B Llama, grouped heads of 128 channels (for measurements
    # at a head size and widths that the three above do not have; usually run with fewer layers)
    "llama-8b": _llama(
        num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
        intermediate_size=14336, vocab_size=128256, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
        max_position_embeddings=8192),
    # two tiny models that differ in every size and option
    "tiny-a": _llama(
        num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, intermediate_size=176,
        vocab_size=512, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=256,
        eos_token_id=2),
    "tiny-b": _llama(
        num_hidden_layers=3, hidden_size=96, num_attention_heads=3, num_key_value_heads=1, intermediate_size=256,
        vocab_size=1000, rope_theta=100000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=512),
}


def preset_names() -> List[str]:
    return sorted(_PRESETS)


def preset(name: str, **overrides) -> Dict[str, Any]:
    """The config.json of a named shape; ``overrides`` replace keys (fewer
    layers for a quick run, a smaller vocabulary for a test)."""
    try:
        config = dict(_PRESETS[name])
    except KeyError:
        raise InvalidInput(f"unknown preset {name!r}; presets are {', '.join(preset_names())}") from None
    config["architectures"] = list(config["architectures"])
    config.update(overrides)
    return config
