"""Loads a model folder's tensors by name.

The parts of a model declare the tensors they read (name, shape); the loader
looks each one up in ``model.safetensors`` (or the shards named by
``model.safetensors.index.json``), checks shape and stored type, and puts it
on the device.  A tensor stored in bfloat16 stays bfloat16 and one stored in
32-bit stays 32-bit; only the 32-bit path widens (exactly, ``bits << 16``:
/root/reference/crates/nnis-model/src/safetensors_loader.rs:610-624).  A table
of integers (a part declares it so) is kept as int32 on either path.
Everything wrong with a folder is reported in one error: missing tensors,
tensors nobody asked for, wrong shapes, unsupported stored types
(the reference's checks: safetensors_loader.rs:711-724,831-874).
"""

from __future__ import annotations

import json
import os
from typing import Dict, List, Sequence

import torch

from ..errors import WeightError
from ..parts.base import TensorSpec
from .safetensors_io import SafetensorsFile

SINGLE = "model.safetensors"
INDEX = "model.safetensors.index.json"
_STORED = {"F32": torch.float32, "BF16": torch.bfloat16}
_STORED_INTEGERS = {"I32": torch.int32, "I64": torch.int64}  # what a table of integers may be stored as
# buffers that older checkpoints carry beside the weights
_IGNORED_SUFFIXES = ("rotary_emb.inv_freq",)


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


def load_weights(model_dir: str, specs: Sequence[TensorSpec], device, widen_to_float32: bool) -> Dict[str, torch.Tensor]:
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
        plan.append((spec.name, source))
    unexpected = sorted(
        name for name in where if name not in consumed and not name.endswith(_IGNORED_SUFFIXES)
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
            lines.append(f"  unsupported stored types ({len(wrong_type)}): " + "; ".join(wrong_type))
        if duplicates:
            lines.append(f"  tensors in more than one shard ({len(duplicates)}): " + "; ".join(sorted(duplicates)))
        raise WeightError("\n".join(lines))

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
            on_device[source] = tensor.contiguous()
        out[name] = on_device[source]
    for handle in files:
        handle.close()
    return out
