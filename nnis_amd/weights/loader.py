"""Loads a model folder's tensors by name.

The parts of a model declare the tensors they read (name, shape); the loader
looks each one up in ``model.safetensors`` (or the shards named by
``model.safetensors.index.json``), checks shape and stored type, and puts it
on the device.  Every tensor's stored type must be the one config.json
declares (``torch_dtype``; safetensors_loader.rs:718-724).  A tensor stored in
bfloat16 stays bfloat16 and one stored in 32-bit stays 32-bit; the 32-bit path
widens (exactly, ``bits << 16``:
/root/reference/crates/nnis-model/src/safetensors_loader.rs:610-624), and
nothing narrows unless the caller asks for it: ``narrow_to_bfloat16`` rounds
32-bit tensors to bfloat16 (nearest, ties to even) as they are loaded, so that
a 32-bit checkpoint under a bfloat16 runtime runs on the matrix cores.  Without
it such a checkpoint keeps its 32-bit weights and every projection takes the
ordered 32-bit product, much slower; the loader says so in one line.  A table
of integers (a part declares it so) is kept as int32 on either path.
Everything wrong with a folder is reported in one error: missing tensors,
tensors nobody asked for, wrong shapes, unsupported stored types
(the reference's checks: safetensors_loader.rs:711-724,831-874).
"""

from __future__ import annotations

import json
import os
import sys
from typing import Dict, List, Optional, Sequence

import torch

from ..errors import WeightError
from ..parts.base import TensorSpec
from .safetensors_io import SafetensorsFile

SINGLE = "model.safetensors"
INDEX = "model.safetensors.index.json"
_STORED = {"F32": torch.float32, "BF16": torch.bfloat16}
_STORED_INTEGERS = {"I32": torch.int32, "I64": torch.int64}  # what a table of integers may be stored as


def _confined(model_dir: str, relative: str) -> str:
    """A shard path named by the index must stay inside the model folder
    (safetensors_loader.rs:301-387)."""
    if os.path.isabs(relative) or ".." in relative.replace("\\", "/").split("/"):
        raise WeightError(f"shard path {relative!r} leaves the model folder")
    path = os.path.join(model_dir, relative)
    real_dir = os.path.realpath(model_dir)
    if os.path.commonpath([real_dir, os.path.realpath(path)]) != real_dir:
        raise WeightError(f"shard path {relative!r} resolves outside the model folder")
    return path


def open_weight_files(model_dir: str) -> List[SafetensorsFile]:
    single = os.path.join(model_dir, SINGLE)
    index = os.path.join(model_dir, INDEX)
    has_single, has_index = os.path.isfile(single), os.path.isfile(index)
    if has_single and has_index:
        # safetensors_loader.rs:389-438
        raise WeightError(f"{model_dir} holds both {SINGLE} and {INDEX}; exactly one is expected")
    if has_single:
        return [SafetensorsFile(single)]
    if has_index:
        try:
            with open(index, "r", encoding="utf-8") as handle:
                weight_map = json.load(handle)["weight_map"]
        except (OSError, ValueError, KeyError) as error:
            raise WeightError(f"invalid {INDEX}: {error}") from None
        shards = sorted(set(weight_map.values()))
        files = []
        for shard in shards:
            path = _confined(model_dir, shard)
            if not os.path.isfile(path):
                raise WeightError(f"shard {shard} named by {INDEX} does not exist")
            files.append(SafetensorsFile(path))
        return files
    raise WeightError(f"{model_dir} holds neither {SINGLE} nor {INDEX}")


_DECLARED = {"float32": "F32", "bfloat16": "BF16"}


def load_weights(model_dir: str, specs: Sequence[TensorSpec], device, widen_to_float32: bool,
                 declared_dtype: Optional[str] = None, narrow_to_bfloat16: bool = False,
                 ignored_suffixes: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """``declared_dtype``: config.json's ``torch_dtype`` ("float32" or
    "bfloat16"; None skips the check, for callers without a config.json).
    ``narrow_to_bfloat16``: round tensors stored in 32-bit to bfloat16 at load
    (not with ``widen_to_float32``).  ``ignored_suffixes``: endings of names
    that a folder of this architecture may hold beside its weights without
    being an error (the model's description names them)."""
    if narrow_to_bfloat16 and widen_to_float32:
        raise WeightError("narrow_to_bfloat16 is for a bfloat16 runtime; the 32-bit path keeps 32-bit weights")
    if declared_dtype is not None and declared_dtype not in _DECLARED:
        raise WeightError(f"config.json declares torch_dtype {declared_dtype!r}; supported are float32 and bfloat16")
    files = open_weight_files(model_dir)
    where: Dict[str, SafetensorsFile] = {}
    duplicates: List[str] = []
    for handle in files:
        for name in handle.names():
            if name in where:
                duplicates.append(name)
            where[name] = handle

    missing: List[str] = []
    wrong_shape: List[str] = []
    wrong_type: List[str] = []
    consumed = set()
    integer_tables = set()  # checkpoint names
    plan = []  # (spec name, checkpoint name)
    seen = set()
    for spec in specs:
        if spec.name in seen:
            continue
        seen.add(spec.name)
        source = spec.name
        if source not in where and spec.fallback is not None and spec.fallback in where:
            source = spec.fallback
        if source not in where:
            missing.append(f"{spec.name} {list(spec.shape)}")
            continue
        consumed.add(source)
        stored, shape = where[source].entries[source]
        if tuple(shape) != tuple(spec.shape):
            wrong_shape.append(f"{source}: expected {list(spec.shape)}, file has {list(shape)}")
            continue
        if spec.init == "index":
            if stored not in _STORED_INTEGERS:
                wrong_type.append(f"{source}: stored as {stored}; a table of integers is stored as I32 or I64")
                continue
            integer_tables.add(source)
        elif stored not in _STORED:
            wrong_type.append(f"{source}: stored as {stored}; supported are F32 and BF16")
            continue
        elif declared_dtype is not None and stored != _DECLARED[declared_dtype]:
            wrong_type.append(f"{source}: stored as {stored}; config.json declares {declared_dtype}")
            continue
        plan.append((spec.name, source))
    unexpected = sorted(
        name for name in where if name not in consumed and not name.endswith(tuple(ignored_suffixes))
    )

    if missing or unexpected or wrong_shape or wrong_type or duplicates:
        lines = [f"model folder {model_dir} does not match the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + "; ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + "; ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        if wrong_type:
            lines.append(f"  wrong stored types ({len(wrong_type)}): " + "; ".join(wrong_type))
        if duplicates:
            lines.append(f"  tensors in more than one shard ({len(duplicates)}): " + "; ".join(sorted(duplicates)))
        raise WeightError("\n".join(lines))

    kept_wide = 0
    on_device: Dict[str, torch.Tensor] = {}  # by checkpoint name: a tied head shares the table's memory
    out: Dict[str, torch.Tensor] = {}
    for name, source in plan:
        if source not in on_device:
            host = where[source].tensor(source)
            if source in integer_tables:
                if host.numel() and (int(host.min()) < -(1 << 31) or int(host.max()) >= (1 << 31)):
                    raise WeightError(f"{source}: a value does not fit the 32-bit integers the table is kept in")
                tensor = host.to(torch.int32).to(device)
            else:
                tensor = host.to(device)
                if widen_to_float32 and tensor.dtype != torch.float32:
                    tensor = tensor.to(torch.float32)
                elif tensor.dtype == torch.float32 and not widen_to_float32:
                    if narrow_to_bfloat16:
                        tensor = tensor.to(torch.bfloat16)  # round to nearest, ties to even
                    else:
                        kept_wide += 1
            on_device[source] = tensor.contiguous()
        out[name] = on_device[source]
    for handle in files:
        handle.close()
    if kept_wide:
        print(f"[nnis_amd] {model_dir}: {kept_wide} tensors are stored in 32-bit and stay so; under bfloat16 their products "
              "take the ordered 32-bit kernel (slow).  narrow_to_bfloat16 / --narrow-to-bfloat16 rounds them at load.",
              file=sys.stderr, flush=True)
    return out
