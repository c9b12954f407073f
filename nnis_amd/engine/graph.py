"""Decode steps replayed from a HIP graph.

A decode step launches a few hundred small kernels; issued one by one from the
host the step is bound by launch overhead, not by the GPU.  For a batch size
(padded up to a bucket) and the plans of the layers' kernels for it (each mixer's own), the step is captured once
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
from typing import Dict, Sequence

import torch

import numpy as np

from ..errors import KernelError
from .batch import RecordedLists, StepContext

BUCKETS = (1, 2, 4, 8, 12, 16, 24, 32, 48, 64)


def bucket(batch: int) -> int:
    for size in BUCKETS:
        if batch <= size:
            return size
    return ((batch + 31) // 32) * 32


class DecodeGraph:
    def __init__(self, engine, padded: int, plan_len: int):
        """``plan_len``: a length whose plans (``DecoderModel.decode_plan`` for ``padded`` sequences) are the
        ones this graph is captured with and replayed for."""
        # not a strong reference: engine -> graphs -> engine would keep both alive until the cycle
        # collector runs, and that may be in the middle of another engine's capture
        self.engine = engine if isinstance(engine, weakref.ProxyTypes) else weakref.proxy(engine)
        self.padded = padded
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
            seq_start=self.rows, seq_pos0=self.meta[2], decode=True, max_new=1, max_len=0, host_new=None, host_pos0=None,
            plan_len=plan_len)
        self.graph = None
        self.logits = None
        self.held = []  # memory the parts' kernels keep between calls, whose addresses the capture baked in: held as long as the graph

    def _forward(self) -> torch.Tensor:
        engine = self.engine
        self.ctx.tables = {}  # the step's tables are made anew by every run (a capture must hold the kernel that makes them)
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
        # A graph that the cycle collector destroys while another is being captured aborts the process: the
        # collector stays off until the capture ends.  (Graphs hold their engine weakly, so an engine that is
        # dropped takes its graphs with it at once; a full collection here cost 30 ms a capture, most of it.)
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph):
                self.logits = self._forward()
        finally:
            if collecting:
                gc.enable()
        # A part's kernels may go through scratch that is kept between calls (the runs of a decode attention's
        # keys meet in one).  The eager run above sized it and the capture baked its address in, so the graph
        # holds what the parts name (``Part.held_buffers``): whatever its keeper does later, a replay never writes
        # into memory that has gone back to the allocator.
        self.held = list(self.engine.model.held_buffers(self.engine.rt))

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


DECODE_GRAPHS_KEPT = 24  # a graph keeps its activations' memory; a batch that shrinks walks through a few buckets and plans


class DecodeGraphs:
    """The graphs of one engine, made on first use; the ``DECODE_GRAPHS_KEPT`` used last are kept."""

    def __init__(self, engine):
        self.engine = weakref.proxy(engine)
        self.graphs: Dict[tuple, DecodeGraph] = {}  # in the order of their last use

    def get(self, batch: int, longest: int) -> DecodeGraph:
        """The graph for ``batch`` sequences, the longest of ``longest`` tokens after the step: one per
        (bucket of the batch, the layers' plans for that bucket and length)."""
        padded = bucket(batch)
        engine = self.engine
        key = (padded, engine.model.decode_plan(padded, longest, engine.rt))
        graph = self.graphs.pop(key, None)
        if graph is None:
            graph = DecodeGraph(engine, padded, longest)
            graph.capture()
            while len(self.graphs) >= DECODE_GRAPHS_KEPT:
                # (the stream may still replay the oldest: it is destroyed only when the GPU has left it)
                torch.cuda.synchronize()
                self.graphs.pop(next(iter(self.graphs)))
        self.graphs[key] = graph  # the most recently used is last
        return graph


# ---------------------------------------------------------------------------------------------
# Prompt steps whose shape comes again
# ---------------------------------------------------------------------------------------------
# A step over a few thousand tokens launches 150 kernels and more; where the model is small the host
# needs as long to launch them as the GPU to run them.  A step's *shape* -- how many sequences it has, how
# many tokens in all (rounded up: ``prompt_rows``), how many logit rows are wanted, and how the model's parts
# plan their launches for it (``DecoderModel.prompt_plan``) -- fixes every launch; tokens, slots,
# positions, how the tokens divide among the sequences and the parts' work lists are data.  The rows
# beyond a step's tokens belong to no sequence (slot -1): every kernel computes them like any row and writes
# nothing of them into the cache, and the parts fill their work lists up with items that do nothing
# (``StepLists``).  The second time a shape comes it runs once from fixed buffers as any step runs, which
# shows which lists its parts ask for, and is then captured into a graph whose kernels read all that data
# from the buffers; from the third time on the step is a copy into the buffers and a replay.  Only shapes of
# up to PREFILL_GRAPH_MOST_TOKENS tokens are kept, the most recently used
# PREFILL_GRAPHS_KEPT of them (a graph keeps its activations' memory), and only where the step's kernels are
# short enough for the host to matter: tokens x width^2 up to PREFILL_GRAPH_MOST_WORK.  Measured, one prompt a
# step, launched against replayed, milliseconds: width 576, 30 layers: 64 tokens 2.27 / 0.83, 256 2.33 / 1.33,
# 1,024 2.41 / 1.64, 2,048 2.42 / 2.24; width 2048, 22 layers: 64 tokens 1.79 / 1.38, 256 2.16 / 2.08, 512
# 2.77 / 2.75, from 1,024 on equal (4.24, 7.28): there the kernels bound the step and a graph would only hold memory.
PREFILL_GRAPH_MOST_TOKENS = 4096
PREFILL_GRAPH_MOST_WORK = 1.5e9
PREFILL_GRAPHS_KEPT = 16


def prompt_rows(total: int) -> int:
    """Rows of the replayed prompt step that takes ``total`` tokens: the next multiple of 64 up to 1,024
    tokens, of 128 up to 2,048, of 256 beyond.  (Parts that plan by a step's size are given this, so that a
    step launched and the same step replayed from a graph's rows take the same kernels.)"""
    unit = 64 if total <= 1024 else (128 if total <= 2048 else 256)
    return ((total + unit - 1) // unit) * unit


class PrefillGraph:
    def __init__(self, engine, batch: int, total: int, wanted: int, plan_len: int):
        """``total``: the rows of the step (``prompt_rows`` of its tokens), ``batch``: its sequences,
        ``plan_len``: a longest sequence for which the parts plan as they do for this shape."""
        self.engine = engine if isinstance(engine, weakref.ProxyTypes) else weakref.proxy(engine)
        self.batch, self.total, self.plan_len = batch, total, plan_len
        # the step's arrays in one buffer, in the order the step function stages them
        self.sizes = [total, total, total, batch, batch + 1, batch, wanted]
        self.lists = None  # the parts' work lists: who makes which, as the first run found them
        self.copied = torch.cuda.Event()
        self.copied.record()
        self.graph = None
        self.logits = None
        self.held = []
        self._lay_out({})

    def _lay_out(self, list_shapes) -> None:
        """One device buffer and one pinned one for the step's arrays and the lists of ``list_shapes``."""
        device = self.engine.rt.device
        self.list_keys = list(list_shapes)
        sizes = self.sizes + [int(np.prod(list_shapes[key])) for key in self.list_keys]
        self.spans, offset = [], 0
        for size in sizes:
            self.spans.append((offset, size))
            offset += size
        self.meta = torch.zeros(offset, dtype=torch.int32, device=device)
        self.host = torch.empty(offset, dtype=torch.int32, pin_memory=True)
        views = [self.meta[o:o + n] for o, n in self.spans]
        self.ids, self.want_rows = views[0], views[6]
        fixed = {key: view.view(list_shapes[key]) for key, view in zip(self.list_keys, views[7:])}
        if self.lists is not None:
            self.lists.fixed = fixed
        # (no host lists: a work list that the first run did not ask for is an error)
        self.ctx = StepContext(
            tokens=self.total, batch=self.batch, tok_slot=views[1], tok_pos=views[2], seq_slot=views[3], seq_start=views[4],
            seq_pos0=views[5], decode=False, max_new=self.total, max_len=self.plan_len, host_new=None, host_pos0=None,
            plan_len=self.plan_len, plan_rows=self.total, lists=self.lists)

    def fill(self, arrays, counts: Sequence[int], first_positions: Sequence[int]) -> None:
        """The step's data into the buffers: ``arrays`` as the step function stages them (ids, slot and position
        of each token, slot, first row and first position of each sequence, wanted rows); ``counts``: the
        tokens each sequence brings.  Rows beyond the tokens get id 0, slot -1, position 0; the parts' lists
        are made anew by those who made them in the first run."""
        self.copied.synchronize()  # the previous copy has left the pinned buffer
        host = self.host.numpy()
        tokens = sum(counts)
        for index, ((offset, size), array) in enumerate(zip(self.spans, arrays)):
            if index < 3:
                host[offset:offset + tokens] = array
                host[offset + tokens:offset + size] = -1 if index == 1 else 0
            else:
                host[offset:offset + size] = array
        for (offset, size), key in zip(self.spans[7:], self.list_keys):
            made = np.asarray(self.lists.makers[key](counts, first_positions, (self.batch, self.total)), dtype=np.int32)
            if made.shape != self.lists.shapes[key]:
                raise KernelError(f"work list {key!r} has shape {made.shape} now, {self.lists.shapes[key]} when the step was captured")
            host[offset:offset + size] = made.reshape(-1)
        self.meta.copy_(self.host, non_blocking=True)
        self.copied.record()

    def _forward(self) -> torch.Tensor:
        engine = self.engine
        self.ctx.tables = {}  # (as for the decode graphs)
        return engine.model.forward(self.ids, self.ctx, engine.cache, self.want_rows, engine.rt)

    def first_run(self, arrays, counts: Sequence[int], first_positions: Sequence[int]):
        """Runs the step from the buffers as any step runs (its parts make their lists, padded to the shape,
        and are recorded), lays the buffers out again with room for those lists, and captures the step's
        launches.  Returns the first run's logits (the caller's to keep), or None if the step cannot run from
        fixed buffers; ``graph`` is None afterwards if it could not be captured."""
        self.fill(arrays, counts, first_positions)
        self.lists = RecordedLists(counts, first_positions, self.engine.rt.device, (self.batch, self.total))
        self.ctx.lists = self.lists
        try:
            logits = self._forward()
        except KernelError:
            return None  # (a part that needs the host's view of the step: the caller runs the step as any step)
        self._lay_out(dict(self.lists.shapes))
        self.fill(arrays, counts, first_positions)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        collecting = gc.isenabled()  # (as for the decode graphs: no graph may be destroyed while one is captured)
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                self.logits = self._forward()
            self.graph = graph
            self.held = list(self.engine.model.held_buffers(self.engine.rt))
        except KernelError:
            # a part that cannot run under capture: the shape goes on being launched
            self.graph = self.logits = None
        finally:
            if collecting:
                gc.enable()
        return logits

    def run(self) -> torch.Tensor:
        """Replays the step on what the buffers hold; the rows returned view the graph's output buffer."""
        self.graph.replay()
        return self.logits


class PrefillGraphs:
    """The prompt-step graphs of one engine: counts how often a shape has come, captures it the second time."""

    def __init__(self, engine):
        self.engine = weakref.proxy(engine)
        self.seen: Dict[tuple, int] = {}
        self.refused = set()  # shapes whose capture failed
        self.graphs: Dict[tuple, PrefillGraph] = {}  # in the order of their last use

    def step(self, key: tuple, arrays, counts: Sequence[int], first_positions: Sequence[int], longest: int):
        """(logits, borrowed) if this step is replayed or captured; None if it is to run as any step.
        ``key``: (sequences, rows, wanted logit rows, the parts' plans); ``longest``: the step's longest
        sequence (one for which the parts plan as the key says)."""
        graph = self.graphs.pop(key, None)
        if graph is not None:
            self.graphs[key] = graph  # the most recently used is last
            graph.fill(arrays, counts, first_positions)
            return graph.run(), True
        if key in self.refused:
            return None
        times = self.seen.get(key, 0) + 1
        self.seen[key] = times
        if len(self.seen) > 1024:
            self.seen.clear()
        if times < 2:
            return None
        batch, total, wanted, _ = key
        graph = PrefillGraph(self.engine, batch, total, wanted, longest)
        logits = graph.first_run(arrays, counts, first_positions)
        if graph.graph is None:
            self.refused.add(key)
            return None if logits is None else (logits, False)
        while len(self.graphs) >= PREFILL_GRAPHS_KEPT:
            # (the stream may still replay the oldest: it is destroyed only when the GPU has left it)
            torch.cuda.synchronize()
            self.graphs.pop(next(iter(self.graphs)))
        self.graphs[key] = graph
        return logits, False
