"""Entry points for callers: load a model folder into an engine."""

from __future__ import annotations

from typing import List, Optional, Sequence, Union

from . import models  # noqa: F401  (registers the architectures)
from .config.llama import read_config_json
from .config.registry import spec_from_config
from .engine.runtime import Runtime
from .engine.step import Engine
from .models.decoder import DecoderModel
from .weights.loader import load_weights


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0", narrow_to_bfloat16: bool = False):
    """Reads config.json, picks the model by its architecture name, loads the
    tensors by name and binds them to the parts.  Returns (model, runtime).
    ``narrow_to_bfloat16``: a checkpoint stored in 32-bit is rounded to
    bfloat16 as it is loaded (only with ``dtype`` bfloat16); without it its
    weights stay 32-bit and take the slow ordered product."""
    raw = read_config_json(model_dir)
    _, spec = spec_from_config(raw)
    rt = Runtime(device=device, dtype=dtype)
    model = DecoderModel(spec)
    model.check(rt)  # a size that the kernels do not take is refused here, before a byte of the weights is read
    weights = load_weights(model_dir, model.tensors(), rt.device, widen_to_float32=rt.is_fp32,
                           declared_dtype=spec.stored_dtype, narrow_to_bfloat16=narrow_to_bfloat16,
                           ignored_suffixes=spec.ignored_tensor_suffixes)
    model.bind(weights, rt)
    return model, rt


def load_engine(model_dir: str, dtype="bfloat16", max_tokens: int = 8192, device="cuda:0",
                max_slots: Optional[int] = None, narrow_to_bfloat16: bool = False) -> Engine:
    model, rt = load_model(model_dir, dtype=dtype, device=device, narrow_to_bfloat16=narrow_to_bfloat16)
    return Engine(model, rt, max_tokens=max_tokens, max_slots=max_slots)


def generate(model, prompts: Sequence[Sequence[int]], max_new_tokens: int = 16, sample: bool = False,
             seed: Union[int, Sequence[int], None] = None, temperature: float = 1.0, top_k: Optional[int] = None,
             top_p: Optional[float] = None, stop_token_ids: Optional[Sequence[int]] = None, dtype="bfloat16",
             device="cuda:0", max_tokens: Optional[int] = None, max_batch: int = 64,
             narrow_to_bfloat16: bool = False) -> List[List[int]]:
    """The Python entry point, with the command line's option names and
    meanings (/root/reference/crates/nnis-cli/src/main.rs:179-365): greedy
    unless ``sample``; ``sample`` requires a seed (one per prompt, or one
    integer for a single prompt); ``temperature``, ``top_k`` and ``top_p``
    apply only with ``sample``.  ``model`` is a model folder or an ``Engine``;
    prompts are token ids.  Stop tokens default to the model's
    ``eos_token_id``.  Returns the new token ids of each prompt, the stop
    token included."""
    from .engine.generate import GenerationRequest, generate as run
    from .errors import InvalidInput
    from .sampling.params import SamplingParams

    if prompts and isinstance(prompts[0], int):
        prompts = [prompts]
    prompts = [list(p) for p in prompts]
    if not sample and (seed is not None or top_k is not None or top_p is not None or temperature != 1.0):
        raise InvalidInput("seed, temperature, top_k and top_p require sample=True")
    seeds: List[Optional[int]] = [None] * len(prompts)
    if sample:
        if seed is None:
            raise InvalidInput("sample=True requires a seed")
        seeds = [seed] if isinstance(seed, int) else list(seed)
        if len(seeds) != len(prompts):
            raise InvalidInput(f"one seed per prompt is required (got {len(prompts)} prompts and {len(seeds)} seeds)")
    if isinstance(model, Engine):
        engine = model
    else:
        need = max_tokens or sum(((len(p) + max_new_tokens + 63) // 64) * 64 for p in prompts)
        engine = load_engine(model, dtype=dtype, max_tokens=need, device=device, narrow_to_bfloat16=narrow_to_bfloat16)
    stops = engine.model.spec.stop_token_ids if stop_token_ids is None else tuple(stop_token_ids)
    requests = [
        GenerationRequest(p, max_new_tokens, stops,
                          SamplingParams(seed=s, temperature=temperature, top_k=top_k, top_p=top_p) if sample else None)
        for p, s in zip(prompts, seeds)
    ]
    return [result.tokens for result in run(engine, requests, max_batch=max_batch)]
