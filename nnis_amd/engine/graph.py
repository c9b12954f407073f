"""Decode steps replayed from a HIP graph.

A decode step launches a few hundred small kernels; issued one by one from the
host the step is bound by launch overhead, not by the GPU.  For a batch size
(padded up to a bucket) and a plan of the attention kernels (splits, waves), the step is captured once
into a graph whose kernels read their token ids, slots and positions from
fixed device buffers; each later step copies three small arrays into those
buffers and replays the graph.  Padding rows carry slot -1: kernels that touch
the cache skip them, the others compute rows nobody reads.

Nothing is memset inside the captured region (buffers come from
``torch.empty``; a graph that needs zeros clears them with a fill kernel).
"""

from __future__ import annotations

import gc
import weakref
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

from .batch import StepContext

BUCKETS = (1, 2, 4, 8, 12, 16, 24, 32, 48, 64)


def bucket(batch: int) -> int:
    for size in BUCKETS:
        if batch <= size:
            return size
    return ((batch + 31) // 32) * 32


class DecodeGraph:
    def __init__(self, engine, padded: int, plan: Tuple[int, int]):
        # not a strong reference: engine -> graphs -> engine would keep both alive until the cycle
        # collector runs, and that may be in the middle of another engine's capture
        self.engine = engine if isinstance(engine, weakref.ProxyTypes) else weakref.proxy(engine)
        self.padded = padded
        splits, waves = plan
        device = engine.rt.device
        # rows: 0 token ids, 1 slots, 2 positions
        self.meta = torch.zeros((3, padded), dtype=torch.int32, device=device)
        self.meta[0].fill_(-1)
        self.meta[1].fill_(-1)
        self.rows = torch.arange(padded + 1, dtype=torch.int32, device=device)
        self.host = torch.empty((3, padded), dtype=torch.int32, pin_memory=True)
        self.copied = torch.cuda.Event()
        self.copied.record()
        self.ctx = StepContext(
            tokens=padded, batch=padded, tok_slot=self.meta[1], tok_pos=self.meta[2], seq_slot=self.meta[1],
            seq_start=self.rows, seq_pos0=self.meta[2], decode=True, max_new=1, max_len=0, splits=splits, waves=waves)
        self.graph = None
        self.logits = None

    def _forward(self) -> torch.Tensor:
        engine = self.engine
        return engine.model.forward(self.meta[0], self.ctx, engine.cache, self.rows[: self.padded], engine.rt)

    def capture(self) -> None:
        # once eagerly on a side stream (loads every kernel), then the capture itself
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._forward()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        # A graph that the cycle collector destroys while another is being captured aborts the process:
        # collect now, and keep the collector off until the capture ends.
        gc.collect()
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph):
                self.logits = self._forward()
        finally:
            if collecting:
                gc.enable()

    def run(self, ids, slots: Sequence[int], positions: Sequence[int], ids_device: torch.Tensor = None) -> torch.Tensor:
        """``ids``: the step's token ids, or None when they are on the device
        already: then row j's id is ``ids_device[j]`` (int32)."""
        count = len(slots)
        self.copied.synchronize()  # the previous copy has left the pinned buffer
        host = self.host.numpy()
        host[0, :count] = ids if ids is not None else -1
        host[1, :count] = slots
        host[2, :count] = positions
        host[0, count:] = -1
        host[1, count:] = -1
        host[2, count:] = 0
        self.meta.copy_(self.host, non_blocking=True)
        self.copied.record()
        if ids is None:
            self.meta[0, :count].copy_(ids_device[:count], non_blocking=True)
        self.graph.replay()
        return self.logits


class DecodeGraphs:
    """The graphs of one engine, made on first use."""

    def __init__(self, engine):
        self.engine = weakref.proxy(engine)
        self.graphs: Dict[Tuple[int, Tuple[int, int]], DecodeGraph] = {}

    def get(self, batch: int, plan: Tuple[int, int]) -> DecodeGraph:
        key = (bucket(batch), plan)
        graph = self.graphs.get(key)
        if graph is None:
            graph = DecodeGraph(self.engine, key[0], plan)
            graph.capture()
            self.graphs[key] = graph
        return graph
