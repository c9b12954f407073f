"""A decoder put together from a ``ModelSpec``: embedding, blocks run in the
order of the schedule, final norm and head.  Nothing here names an
architecture; which parts exist and how they are sized is the spec's business.
"""

from __future__ import annotations

from typing import Any, Dict, List, Tuple

import torch

from ..parts import build_part
from ..parts.base import TensorSpec
from .spec import ModelSpec


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.positions = {name: build_part("position", description) for name, description in spec.positions.items()}
        self.embedding = build_part("embedding", spec.embedding)
        self.layers = [build_part("block", description, positions=self.positions) for description in spec.layers]
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.bound = False
        self._plans = {}
        self._prompt_plans = {}

    # ---- weights -------------------------------------------------------------
    def parts(self):
        return [self.embedding, *self.positions.values(), *self.layers, self.final_norm, self.head]

    def tensors(self) -> List[TensorSpec]:
        out, seen = [], set()
        for part in self.parts():
            for tensor in part.tensors():
                if tensor.name not in seen:
                    seen.add(tensor.name)
                    out.append(tensor)
        return out

    def bind(self, weights: Dict[str, torch.Tensor], rt) -> None:
        parts = self.parts()
        for part in parts:
            part.bind(weights, rt)
        # a tensor that two parts share (a tied head's table) is kept once: whoever packed it offers the copy
        for owner in parts:
            for source, packed in owner.packed_sources():
                for part in parts:
                    if part is not owner:
                        part.adopt_packed(source, packed)
        self.bound = True

    def step_weight_bytes(self) -> int:
        """Bytes of weights a decode step reads: every layer each time the
        schedule runs it, the head, and no embedding table (a row per token)."""
        total = sum(self.layers[entry.layer].weight_bytes() for entry in self.spec.schedule)
        return total + self.final_norm.weight_bytes() + self.head.weight_bytes()

    def graph_safe(self) -> bool:
        """True when a step's kernels read tokens, slots and positions from
        device memory only, so that a captured step can be replayed."""
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    def check(self, rt) -> None:
        """Every part's own check of its sizes against the kernels (``Part.check``): raises ``Unsupported``."""
        for part in self.parts():
            part.check(rt)

    def held_buffers(self, rt):
        """What the parts' kernels keep between calls and a captured step has baked in (``Part.held_buffers``)."""
        return [buffer for part in self.parts() for buffer in part.held_buffers(rt)]

    def prompt_plan(self, batch: int, rows: int, longest: int, rt):
        """The plans of every run of the schedule for a step of prompts (``Part.prompt_plan``)."""
        key = (batch, rows, longest)
        plans = self._prompt_plans.get(key)
        if plans is None:
            if len(self._prompt_plans) > 4096:
                self._prompt_plans.clear()
            plans = self._prompt_plans[key] = tuple(
                self.layers[entry.layer].prompt_plan(batch, rows, longest, rt) for entry in self.spec.schedule)
        return plans

    def decode_plan(self, batch: int, longest: int, rt):
        """The plans of every run of the schedule for a step of one token
        each (``Block.decode_plan``): each layer plans for its own heads and
        sizes.  Plans depend on a length through its pages only."""
        key = (batch, (longest + 63) // 64)
        plans = self._plans.get(key)
        if plans is None:
            if len(self._plans) > 4096:
                self._plans.clear()
            plans = self._plans[key] = tuple(self.layers[entry.layer].decode_plan(batch, longest, rt) for entry in self.spec.schedule)
        return plans

    # ---- cache ---------------------------------------------------------------
    def cache_requests(self) -> Tuple[List[Tuple[int, Any]], Dict[int, int]]:
        requests, shared = [], {}
        for index, entry in enumerate(self.spec.schedule):
            if entry.reads_cache_of is None:
                requests.append((index, self.layers[entry.layer].cache_request()))
            else:
                shared[index] = entry.reads_cache_of
        return requests, shared

    # ---- forward -------------------------------------------------------------
    def forward(self, ids: torch.Tensor, ctx, cache, want_rows: torch.Tensor, rt) -> torch.Tensor:
        """ids: int32 [tokens] on the device; want_rows: int32 indices of the
        packed tokens whose logits are asked for.  Returns float32
        [len(want_rows), vocab]."""
        x = self.embedding.forward(ids, ctx.tokens, rt)
        for position in self.positions.values():
            x = position.embed(x, ctx, rt)
        stream = (x, None)
        schedule = self.spec.schedule
        for index, entry in enumerate(schedule):
            layer = self.layers[entry.layer]
            # a block may prepare the first norm of the block that comes next, if that block shows it one
            following = None
            if index + 1 < len(schedule) and getattr(layer, "entry_norm", None) is not None:
                following = getattr(self.layers[schedule[index + 1].layer], "entry_norm", None)
            if following is not None:
                stream = layer.forward(stream, ctx, cache.view(index), rt, following=following)
            else:
                stream = layer.forward(stream, ctx, cache.view(index), rt)
        x, pending = stream
        if want_rows.shape[0] == 0:
            return rt.empty(0, self.spec.vocab_size, dtype=torch.float32)
        if pending is None:
            normed = self.final_norm.forward(x, rt, rows=want_rows)
        else:
            normed = self.final_norm.add_forward(x, pending, rt, rows=want_rows)
        return self.head.forward(normed, rt)
