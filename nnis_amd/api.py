"""Entry points for callers: load a model folder into an engine."""

from __future__ import annotations

from typing import Optional

from . import models  # noqa: F401  (registers the architectures)
from .config.llama import read_config_json
from .config.registry import spec_from_config
from .engine.runtime import Runtime
from .engine.step import Engine
from .models.decoder import DecoderModel
from .weights.loader import load_weights


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0"):
    """Reads config.json, picks the model by its architecture name, loads the
    tensors by name and binds them to the parts.  Returns (model, runtime)."""
    raw = read_config_json(model_dir)
    _, spec = spec_from_config(raw)
    rt = Runtime(device=device, dtype=dtype)
    model = DecoderModel(spec)
    weights = load_weights(model_dir, model.tensors(), rt.device, widen_to_float32=rt.is_fp32)
    model.bind(weights, rt)
    return model, rt


def load_engine(model_dir: str, dtype="bfloat16", max_tokens: int = 8192, device="cuda:0",
                max_slots: Optional[int] = None) -> Engine:
    model, rt = load_model(model_dir, dtype=dtype, device=device)
    return Engine(model, rt, max_tokens=max_tokens, max_slots=max_slots)
