"""A model as data: which parts, with which parameters, run in which order.

An architecture's builder turns its typed configuration into one
``ModelSpec``.  Everything after that (loading, the cache layout, the step)
reads only the spec, so another architecture is another builder and, where it
needs them, other part kinds.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from ..errors import InvalidInput


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``layer`` indexes ``ModelSpec.layers`` and may
    appear in several entries (shared weights).  ``reads_cache_of`` is the
    index of an earlier schedule entry whose cache this run reads instead of
    keeping one of its own (it then writes nothing)."""

    layer: int
    reads_cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    architecture: str
    width: int
    vocab_size: int
    max_positions: int
    stored_dtype: str  # "float32" or "bfloat16": the type random weights are written in
    embedding: Dict[str, Any]
    positions: Dict[str, Dict[str, Any]]  # named position encodings, built once and shared
    layers: List[Dict[str, Any]]  # block descriptions
    schedule: List[ScheduleEntry]
    final_norm: Dict[str, Any]
    head: Dict[str, Any]
    stop_token_ids: Tuple[int, ...] = ()
    # endings of tensor names that a folder may hold beside the weights without being an error
    ignored_tensor_suffixes: Tuple[str, ...] = ()
    config_json: Dict[str, Any] = field(default_factory=dict)  # what a model folder's config.json holds

    def validate(self) -> None:
        if not self.schedule:
            raise InvalidInput("a model needs at least one schedule entry")
        for index, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise InvalidInput(f"schedule entry {index} names layer {entry.layer}, but there are {len(self.layers)}")
            if entry.reads_cache_of is not None:
                if not 0 <= entry.reads_cache_of < index:
                    raise InvalidInput(
                        f"schedule entry {index} reads the cache of entry {entry.reads_cache_of}, which does not run before it"
                    )
                if self.schedule[entry.reads_cache_of].reads_cache_of is not None:
                    raise InvalidInput(
                        f"schedule entry {index} reads the cache of entry {entry.reads_cache_of}, which keeps none of its own"
                    )
