"""Random-weights mode: writes a model folder (config.json, model.safetensors)
from a configuration and a seed.  Every matrix is N(0, 0.02), every norm
gain 1 + N(0, 0.01) and every table of integers uniform in its range, drawn in the order the model declares its tensors from
one seeded generator.  The reference has no such mode; it downloads a pinned
random checkpoint (/root/reference/tools/tiny_random_llama_fixture.py:29-31).
"""

from __future__ import annotations

import json
import os
from typing import Any, Dict

import torch

from typing import Callable

from ..config.registry import spec_from_config
from ..errors import InvalidInput
from .safetensors_io import write_safetensors

_STORED = {"float32": torch.float32, "bfloat16": torch.bfloat16}

# Init rules, by the name a part gives in ``TensorSpec.init``.  A rule draws one tensor:
# ``rule(spec, generator, dtype) -> tensor`` (``dtype``: the type the model's floats are stored in; a rule for
# integers ignores it).  A part with a tensor of another kind (a bias of zeros, a log-spaced constant) registers
# its own rule beside the part; nothing here knows the rules by name.
_INIT_RULES: Dict[str, Callable[[Any, torch.Generator, torch.dtype], torch.Tensor]] = {}


def register_init_rule(name: str, rule: Callable[[Any, torch.Generator, torch.dtype], torch.Tensor], replace: bool = False) -> None:
    if name in _INIT_RULES and not replace:
        raise InvalidInput(f"init rule {name!r} is already registered")
    _INIT_RULES[name] = rule


def registered_init_rules():
    return sorted(_INIT_RULES)


def _noise(spec, generator) -> torch.Tensor:
    return torch.randn(tuple(spec.shape), generator=generator, dtype=torch.float32)


def _index(spec, generator, dtype) -> torch.Tensor:
    if not spec.high or spec.high <= 0:
        raise InvalidInput(f"tensor {spec.name}: a table of integers needs the end of its range (high)")
    return torch.randint(0, int(spec.high), tuple(spec.shape), generator=generator, dtype=torch.int32)


register_init_rule("matrix", lambda spec, generator, dtype: (0.02 * _noise(spec, generator)).to(dtype))
register_init_rule("gain", lambda spec, generator, dtype: (1.0 + 0.01 * _noise(spec, generator)).to(dtype))
register_init_rule("zeros", lambda spec, generator, dtype: torch.zeros(tuple(spec.shape), dtype=dtype))
register_init_rule("index", _index)


def write_random_model(model_dir: str, raw_config: Dict[str, Any], seed: int) -> str:
    """``raw_config`` is what config.json will hold."""
    from ..models.decoder import DecoderModel

    _, spec = spec_from_config(raw_config)
    model = DecoderModel(spec)
    dtype = _STORED.get(spec.stored_dtype)
    if dtype is None:
        raise InvalidInput(f"random weights are written as float32 or bfloat16, not {spec.stored_dtype!r}")
    generator = torch.Generator(device="cpu")
    generator.manual_seed(int(seed))

    def draw():
        done = set()
        for tensor in model.tensors():
            if tensor.name in done or tensor.fallback is not None:
                continue  # a tensor with a stand-in (tied head) is not drawn
            done.add(tensor.name)
            rule = _INIT_RULES.get(tensor.init)
            if rule is None:
                raise InvalidInput(f"tensor {tensor.name}: unknown init rule {tensor.init!r}; registered: "
                                   f"{', '.join(registered_init_rules())}")
            yield tensor.name, rule(tensor, generator, dtype)

    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(spec.config_json or raw_config, handle, indent=2)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), draw(), {"format": "pt", "seed": str(seed)})
    return model_dir
