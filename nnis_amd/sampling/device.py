"""Token selection on the device for a batch of logit rows: argmax for greedy
rows, the sampling kernel for seeded rows.  Each sequence's generator state and
its sampling options live in the cache's per-slot state regions, so a
sequence's draws do not depend on what else is in the batch
(/root/reference/crates/nnis-model/src/session_batch.rs:7-8) and a step's
selection needs nothing from the host but the rows' slots."""

from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..errors import InvalidInput
from .params import SamplingParams

RNG_REGION = "sampler.rng"
# the options of a sequence that samples, set when it starts (``DeviceSelector.start``)
OPTION_REGIONS = {"sampler.temperature": torch.float32, "sampler.top_k": torch.int32, "sampler.top_p": torch.float32}


class PendingTokens:
    """Tokens that a selection kernel has been asked for: on the device at
    once (in stream order), on the host when ``result`` returns."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, event):
        self.device = device
        self._host = host
        self._event = event

    def result(self) -> List[int]:
        self._event.synchronize()
        tokens = self._host.tolist()
        for row, token in enumerate(tokens):
            if token < 0:  # what the sampling kernel leaves in place of a token it will not draw
                raise InvalidInput(f"sampling refused row {row}: a logit is not finite")
        return tokens


class DeviceSelector:
    def __init__(self, engine):
        self.engine = engine
        self.rt = engine.rt
        self.vocab_size = engine.vocab_size
        cache = engine.cache
        for name, dtype in {RNG_REGION: torch.int64, **OPTION_REGIONS}.items():
            if name not in cache.state_regions:
                cache.add_state_region(name, (), dtype)
        self.rng = cache.state_regions[RNG_REGION]
        self.temperature, self.top_k, self.top_p = (cache.state_regions[name] for name in OPTION_REGIONS)
        self._weights = None
        self._pairs = [None, None]  # (device, pinned host, event) of select_start, used in turn
        self._turn = 0
        self._row_slots = (None, None)  # the slots of the rows that sample (-1: a greedy row), as last asked for, and on the device

    def start(self, slot: int, params: Optional[SamplingParams]) -> None:
        """Called when a sequence starts: seeds its generator and keeps its options with its slot."""
        if params is not None:
            params.validate(self.vocab_size)
            seed = params.seed if params.seed < (1 << 63) else params.seed - (1 << 64)
            self.rng[slot] = seed
            self.temperature[slot] = float(params.temperature)
            self.top_k[slot] = int(params.top_k or 0)
            self.top_p[slot] = float(params.top_p or 0.0)

    def _sampling_rows(self, slots: Sequence[int], params: Sequence[Optional[SamplingParams]]) -> torch.Tensor:
        """int32 on the device: a row's slot if it samples, -1 if it is greedy.  Copied only when it changes
        (a batch's rows change when a sequence ends, not from step to step)."""
        key = tuple(int(s) if p is not None else -1 for s, p in zip(slots, params))
        if self._row_slots[0] != key:
            self._row_slots = (key, torch.tensor(key, dtype=torch.int32, device=self.rt.device))
        return self._row_slots[1]

    def select_start(self, logits: torch.Tensor, slots: Sequence[int], params: Sequence[Optional[SamplingParams]]):
        """The selection of one token per row of ``logits`` (float32 [rows,
        vocab] on the device) is put on the stream and the copy of the tokens
        to the host behind it; nothing waits.  ``params[j]`` says whether row j
        samples (its options are those its sequence started with) or is greedy
        (None).  Returns a ``PendingTokens``: the tokens on the device (for a
        step that starts before the host has read them) and ``result()``, which
        waits for the copy.  Two results may be outstanding at a time: the
        third call reuses the first's buffers."""
        rows = logits.shape[0]
        ops = self.rt.ops
        self._turn ^= 1
        pair = self._pairs[self._turn]
        if pair is None or pair[0].numel() < rows:
            size = max(rows, 64)
            pair = self._pairs[self._turn] = (torch.empty(size, dtype=torch.int32, device=self.rt.device),
                                              torch.empty(size, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
        device, host, event = pair
        ops.argmax(logits, device[:rows])
        if any(p is not None for p in params):
            if self._weights is None or self._weights.shape[0] < rows:
                self._weights = torch.empty((max(rows, 8), self.vocab_size), dtype=torch.float64, device=self.rt.device)
            # the rows that sample are written over; a greedy row keeps its argmax
            ops.sample(logits, self._weights, self._sampling_rows(slots, params), self.rng, self.temperature, self.top_k,
                       self.top_p, device[:rows], by_slot=True, best=device[:rows])
        host[:rows].copy_(device[:rows], non_blocking=True)
        event.record()
        return PendingTokens(device[:rows], host[:rows], event)

    def select(self, logits: torch.Tensor, slots: Sequence[int], params: Sequence[Optional[SamplingParams]]) -> List[int]:
        """One token per row of ``logits``, on the host."""
        return self.select_start(logits, slots, params).result()
