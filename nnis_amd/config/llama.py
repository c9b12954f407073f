"""Typed configuration of the Llama decoder, read from its own config.json keys.

Keys, defaults and rejections follow the reference's Hugging Face reader
(/root/reference/crates/nnis-model/src/safetensors_loader.rs:66-93 for the
fields, :136-210 for the checks) and its shape validation
(/root/reference/crates/nnis-model/src/config.rs:38-101).

Deliberate differences from the reference, each stated where it applies:
  * ``head_dim`` is read when the file gives it (the reference derives it as
    hidden_size / num_attention_heads and never reads the key, config.rs:103);
  * ``eos_token_id`` may be a list: the generation loop stops on a set.
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import Any, Dict, Tuple

from ..errors import InvalidInput, Unsupported

_DTYPES = {"float32": "float32", "f32": "float32", "bfloat16": "bfloat16", "bf16": "bfloat16"}

_REQUIRED = (
    "architectures",
    "model_type",
    "vocab_size",
    "hidden_size",
    "intermediate_size",
    "num_hidden_layers",
    "num_attention_heads",
    "max_position_embeddings",
    "rms_norm_eps",
    "rope_theta",
    "hidden_act",
    "torch_dtype",
)


def _positive_int(raw: Dict[str, Any], key: str) -> int:
    value = raw[key]
    if isinstance(value, bool) or not isinstance(value, int):
        raise InvalidInput(f"config.json {key} must be an integer; got {value!r}")
    if value <= 0:
        # config.rs:39-54: every size must be non-zero
        raise InvalidInput(f"model config {key} must be non-zero; got {value}")
    return value


def _positive_float(raw: Dict[str, Any], key: str) -> float:
    value = raw[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise InvalidInput(f"config.json {key} must be a number; got {value!r}")
    value = float(value)
    if not math.isfinite(value) or value <= 0.0:
        # config.rs:80-91
        raise InvalidInput(f"{key} must be finite and positive; got {value}")
    return value


@dataclass(frozen=True)
class LlamaConfig:
    """Every size and constant of one Llama model.  Nothing here has a default
    that stands for a value config.json must give."""

    architecture: str
    model_type: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    hidden_act: str
    tie_word_embeddings: bool
    torch_dtype: str
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)

    # ---- derived sizes -------------------------------------------------
    @property
    def q_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        # config.rs:107-111 key_value_width
        return self.num_key_value_heads * self.head_dim

    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def attention_topology(self) -> str:
        """MHA / GQA / MQA as the reference's capability record names them
        (/root/reference/crates/nnis-model/src/decoder_capabilities.rs:10-121)."""
        if self.num_key_value_heads == self.num_attention_heads:
            return "MHA"
        if self.num_key_value_heads == 1:
            return "MQA"
        return "GQA"

    def capability_record(self) -> str:
        """The reference's canonical capability record, line for line
        (decoder_capabilities.rs:72-91; its fixtures for the two pinned
        checkpoints: exact_checkpoint_spec.rs:10-30)."""
        topology = {"MHA": "multi_head", "GQA": "grouped_query", "MQA": "multi_query"}[self.attention_topology()]
        stored = {"float32": "f32", "bfloat16": "bf16"}[self.torch_dtype]
        return (f"NNIS-DECODER-CAPABILITY-V1\nattention={topology}\nrope=llama_rotate_half_unscaled\nmlp=swiglu_silu\n"
                f"weight_dtype={stored}\nq_heads={self.num_attention_heads}\nkv_heads={self.num_key_value_heads}\n"
                f"head_dim={self.head_dim}\n")

    def describe(self) -> Dict[str, Any]:
        """What this configuration asks of the engine, with the sizes a caller
        plans memory by: parameters, bytes of weights as stored, bytes of cache
        a token takes in each runtime type."""
        h, inner, layers = self.hidden_size, self.intermediate_size, self.num_hidden_layers
        per_layer = (self.q_width + 2 * self.kv_width) * h + h * self.q_width + 3 * h * inner + 2 * h
        table = self.vocab_size * h
        parameters = layers * per_layer + h + table * (1 if self.tie_word_embeddings else 2)
        stored_bytes = 2 if self.torch_dtype == "bfloat16" else 4
        cache_elements = 2 * layers * self.kv_width
        return {
            "architecture": self.architecture,
            "attention": self.attention_topology(),
            "query_heads": self.num_attention_heads,
            "key_value_heads": self.num_key_value_heads,
            "group_size": self.group_size,
            "head_dim": self.head_dim,
            "position_encoding": "rotary, rotate-half, unscaled",
            "rope_theta": self.rope_theta,
            "feed_forward": "gated (SiLU on the gate)",
            "norm": "RMSNorm",
            "rms_norm_eps": self.rms_norm_eps,
            "layers": layers,
            "width": h,
            "inner": inner,
            "vocab_size": self.vocab_size,
            "max_positions": self.max_position_embeddings,
            "tied_head": self.tie_word_embeddings,
            "stored_dtype": self.torch_dtype,
            "runtime_dtypes": ["bfloat16", "float32"],
            "parameters": parameters,
            "weight_bytes": parameters * stored_bytes,
            "cache_bytes_per_token": {"bfloat16": 2 * cache_elements, "float32": 4 * cache_elements},
            "stop_token_ids": list(self.eos_token_ids),
            "capability_record": self.capability_record(),
        }

    # ---- construction --------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "LlamaConfig":
        missing = [key for key in _REQUIRED if key not in raw]
        if missing:
            raise InvalidInput("config.json is missing required key(s): " + ", ".join(missing))

        architectures = raw["architectures"]
        model_type = raw["model_type"]
        if (
            not isinstance(architectures, list)
            or len(architectures) != 1
            or architectures[0] != "LlamaForCausalLM"
            or model_type != "llama"
        ):
            # safetensors_loader.rs:137-145
            raise Unsupported(
                f"unsupported architecture {architectures!r} / model_type {model_type!r}; "
                "this configuration class reads only LlamaForCausalLM with model_type=llama"
            )
        if raw["hidden_act"] != "silu":
            # safetensors_loader.rs:146-151
            raise Unsupported(
                f"unsupported hidden_act {raw['hidden_act']!r}; the gated feed-forward here is silu/SwiGLU"
            )
        if raw.get("attention_bias", False) or raw.get("mlp_bias", False):
            # safetensors_loader.rs:152-156
            raise Unsupported("attention_bias / mlp_bias tensors are not supported")
        if raw.get("rope_interleaved", False) or raw.get("rope_scaling") is not None:
            # safetensors_loader.rs:157-161
            raise Unsupported("interleaved or scaled RoPE (rope_interleaved / rope_scaling) is not supported")
        dtype = _DTYPES.get(raw["torch_dtype"])
        if dtype is None:
            # safetensors_loader.rs:163-171
            raise Unsupported(
                f"unsupported torch_dtype {raw['torch_dtype']!r}; supported source dtypes are float32 and bfloat16"
            )

        sizes = {
            key: _positive_int(raw, key)
            for key in (
                "vocab_size",
                "hidden_size",
                "intermediate_size",
                "num_hidden_layers",
                "num_attention_heads",
                "max_position_embeddings",
            )
        }
        heads = sizes["num_attention_heads"]
        if raw.get("num_key_value_heads") is None:
            kv_heads = heads  # safetensors_loader.rs:177-179
        else:
            kv_heads = _positive_int(raw, "num_key_value_heads")
        if raw.get("head_dim") is None:
            if sizes["hidden_size"] % heads != 0:
                # config.rs:62-67
                raise InvalidInput(
                    f"hidden_size {sizes['hidden_size']} is not divisible by num_attention_heads {heads}"
                )
            head_dim = sizes["hidden_size"] // heads
        else:
            head_dim = _positive_int(raw, "head_dim")
        if heads % kv_heads != 0:
            # config.rs:68-73
            raise InvalidInput(
                f"num_attention_heads {heads} is not divisible by num_key_value_heads {kv_heads}"
            )
        if head_dim % 2 != 0:
            # config.rs:74-79
            raise InvalidInput(f"rotary head dimension must be even; got {head_dim}")

        eos_raw = raw.get("eos_token_id")
        if eos_raw is None:
            eos: Tuple[int, ...] = ()
        elif isinstance(eos_raw, int) and not isinstance(eos_raw, bool):
            eos = (eos_raw,)
        elif isinstance(eos_raw, list) and all(isinstance(v, int) and not isinstance(v, bool) for v in eos_raw):
            eos = tuple(eos_raw)
        else:
            raise InvalidInput(f"eos_token_id must be an integer or a list of integers; got {eos_raw!r}")
        for token in eos:
            if token < 0 or token >= sizes["vocab_size"]:
                # config.rs:55-61
                raise InvalidInput(
                    f"eos_token_id {token} is out of range for vocabulary {sizes['vocab_size']}"
                )

        tie = raw.get("tie_word_embeddings", False)  # default false: safetensors_loader.rs:82-83
        if not isinstance(tie, bool):
            raise InvalidInput(f"tie_word_embeddings must be true or false; got {tie!r}")

        return cls(
            architecture=architectures[0],
            model_type=model_type,
            vocab_size=sizes["vocab_size"],
            hidden_size=sizes["hidden_size"],
            intermediate_size=sizes["intermediate_size"],
            num_hidden_layers=sizes["num_hidden_layers"],
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            max_position_embeddings=sizes["max_position_embeddings"],
            rms_norm_eps=_positive_float(raw, "rms_norm_eps"),
            rope_theta=_positive_float(raw, "rope_theta"),
            hidden_act=raw["hidden_act"],
            tie_word_embeddings=tie,
            torch_dtype=dtype,
            eos_token_ids=eos,
        )

    def to_dict(self) -> Dict[str, Any]:
        """The config.json this configuration is read back from."""
        out: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "hidden_act": self.hidden_act,
            "tie_word_embeddings": self.tie_word_embeddings,
            "torch_dtype": self.torch_dtype,
        }
        if len(self.eos_token_ids) == 1:
            out["eos_token_id"] = self.eos_token_ids[0]
        elif self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as handle:
            raw = json.load(handle)
    except FileNotFoundError:
        raise InvalidInput(f"{path} does not exist") from None
    except json.JSONDecodeError as error:
        raise InvalidInput(f"invalid config.json at {path}: {error}") from None
    if not isinstance(raw, dict):
        raise InvalidInput(f"config.json at {path} must hold a JSON object")
    return raw
