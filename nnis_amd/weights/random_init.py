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

from ..config.registry import spec_from_config
from ..errors import InvalidInput
from .safetensors_io import write_safetensors

_STORED = {"float32": torch.float32, "bfloat16": torch.bfloat16}


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
            if tensor.init == "index":
                if not tensor.high or tensor.high <= 0:
                    raise InvalidInput(f"tensor {tensor.name}: a table of integers needs the end of its range (high)")
                yield tensor.name, torch.randint(0, int(tensor.high), tuple(tensor.shape), generator=generator, dtype=torch.int32)
                continue
            noise = torch.randn(tensor.shape, generator=generator, dtype=torch.float32)
            if tensor.init == "gain":
                value = 1.0 + 0.01 * noise
            elif tensor.init == "matrix":
                value = 0.02 * noise
            else:
                raise InvalidInput(f"tensor {tensor.name}: unknown init rule {tensor.init!r}")
            yield tensor.name, value.to(dtype)

    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(spec.config_json or raw_config, handle, indent=2)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), draw(), {"format": "pt", "seed": str(seed)})
    return model_dir
