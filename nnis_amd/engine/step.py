"""The step function: runs exactly the tokens it is given, as one batch, from
the cache that earlier steps left, and returns the logits at the wanted
places.  Sequences of a step may have any lengths; a prompt goes in one step,
then one token at a time.  The reference's two entry points, ``prefill`` and
``decode_one`` (/root/reference/crates/nnis-model/src/runtime.rs:756-790), are
both this call; its validation rules (runtime.rs:1134-1163) are kept, and a
refused step changes nothing.
"""

from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache import SequenceCache
from ..errors import InvalidInput
from .batch import StepContext, StepEntry
from .graph import PREFILL_GRAPH_MOST_TOKENS, PREFILL_GRAPH_MOST_WORK, PrefillGraphs, prompt_rows


class Engine:
    def __init__(self, model, rt, max_tokens: int, max_slots: Optional[int] = None, use_graphs: Optional[bool] = None):
        if not model.bound:
            raise InvalidInput("the model has no weights bound; load it first")
        self.model = model
        self.rt = rt
        model.check(rt)  # (a model that was not loaded through ``load_model``: sizes the kernels refuse stop here)
        self.vocab_size = model.spec.vocab_size
        self.max_positions = model.spec.max_positions
        requests, shared = model.cache_requests()
        self.cache = SequenceCache(requests, shared, max_tokens, model.spec.max_positions, rt.dtype, rt.device, max_slots)
        self._staging = None
        self._staging_dev = None
        self._staged = None  # recorded behind the staging copy
        # decode steps are replayed from HIP graphs when every part of the model
        # runs only kernels that read the step's metadata from device memory
        self._borrowed = False
        self.use_graphs = model.graph_safe() if use_graphs is None else (use_graphs and model.graph_safe())
        self._graphs = None
        self._prefill_graphs = None  # prompt steps whose shape comes again
        # A step's positions index the rotation tables on the device, where nothing can refuse them: the tables
        # reach as far as the cache lets a sequence grow, so the check of the lengths before a step covers both.
        for name, position in model.positions.items():
            tables = position.rotary()
            if tables is not None and tables.cos.shape[0] < self.max_positions:
                raise InvalidInput(f"position encoding {name!r} has tables for {tables.cos.shape[0]} positions; "
                                   f"the model's sequences may reach {self.max_positions}")

    # ---- sequences -----------------------------------------------------------
    def start_sequence(self) -> int:
        return self.cache.acquire()

    def end_sequence(self, slot: int) -> None:
        self.cache.release(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    def truncate(self, slot: int, length: int) -> None:
        """Shortens a sequence to its first ``length`` tokens; the next step
        appends there.  Pages beyond go back to the cache at once."""
        self.cache.truncate(slot, length)

    def reset(self, slot: int) -> None:
        """Empties a sequence's slot without giving the slot back."""
        self.cache.reset(slot)

    def free_slots(self) -> int:
        return self.cache.slots.free

    def free_pages(self) -> int:
        groups = self.cache.kv_groups
        return min(g.table.pool.free for g in groups) if groups else 1 << 30

    # ---- one step ------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]):
        if not entries:
            raise InvalidInput("a step needs at least one sequence")
        seen = set()
        growth = {}
        arrays = []  # each entry's token ids, as checked
        for entry in entries:
            if entry.slot in seen:
                raise InvalidInput(f"slot {entry.slot} appears twice in one step")
            seen.add(entry.slot)
            self.cache.length(entry.slot)  # raises if the slot is not held
            count = len(entry.tokens)
            if count == 0:
                raise InvalidInput(f"slot {entry.slot}: a step needs at least one token per sequence")
            try:
                ids = np.asarray(entry.tokens, dtype=np.int64)  # a prompt of thousands: checked as an array, not one by one
            except (TypeError, ValueError, OverflowError):
                raise InvalidInput(f"slot {entry.slot}: token ids must be integers") from None
            if ids.ndim != 1 or int(ids.min()) < 0 or int(ids.max()) >= self.vocab_size:
                bad = next((t for t in entry.tokens if not 0 <= int(t) < self.vocab_size), entry.tokens)
                # runtime.rs:1155-1163
                raise InvalidInput(f"token id {bad} is out of range for vocabulary {self.vocab_size}")
            arrays.append(ids)
            if entry.want is not None and len(entry.want):
                places = np.asarray(entry.want, dtype=np.int64)
                if int(places.min()) < 0 or int(places.max()) >= count:
                    place = next(p for p in entry.want if not 0 <= int(p) < count)
                    raise InvalidInput(f"slot {entry.slot}: wanted place {place} is not among its {count} tokens")
            growth[entry.slot] = count
        self.cache.check_room(growth)
        return growth, arrays

    def _stage(self, arrays: List[np.ndarray]) -> List[torch.Tensor]:
        """One pinned buffer, one copy to the device, views per array."""
        total = sum(a.size for a in arrays)
        if self._staging is None or self._staging.numel() < total:
            size = max(1024, 1 << (total - 1).bit_length())
            self._staging = torch.empty(size, dtype=torch.int32, pin_memory=True)
            self._staging_dev = torch.empty(size, dtype=torch.int32, device=self.rt.device)
            self._staged = torch.cuda.Event()
        else:
            self._staged.synchronize()  # the pinned buffer is reused: the previous step's copy has left it
        host = self._staging.numpy()
        offset = 0
        spans = []
        for array in arrays:
            host[offset:offset + array.size] = array
            spans.append((offset, array.size))
            offset += array.size
        # the previous step's kernels may still read the device buffer: the
        # copy is ordered after them on the same stream
        self._staging_dev[:total].copy_(self._staging[:total], non_blocking=True)
        self._staged.record()
        return [self._staging_dev[o:o + n] for o, n in spans]

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Returns float32 logits [wanted places, vocab], in the order of the
        entries and of each entry's ``want``.  The result is the caller's to keep."""
        logits = self.step_view(entries)
        return logits.clone() if self._borrowed else logits

    def step_view(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """As ``step``, but the rows may view a buffer that the next step
        overwrites: for callers that read them at once (the generation loop)."""
        self._borrowed = False
        self.rt.check_current()
        if self.use_graphs and entries and all(len(e.tokens) == 1 for e in entries):
            return self._decode_step(entries)
        growth, token_arrays = self._validate(entries)
        pos0 = [self.cache.length(e.slot) for e in entries]
        counts = [len(e.tokens) for e in entries]
        total = sum(counts)
        ids = np.empty(total, dtype=np.int32)
        tok_slot = np.empty(total, dtype=np.int32)
        tok_pos = np.empty(total, dtype=np.int32)
        seq_start = np.zeros(len(entries) + 1, dtype=np.int32)
        want_rows: List[int] = []
        row = 0
        for index, entry in enumerate(entries):
            n = counts[index]
            ids[row:row + n] = token_arrays[index]
            tok_slot[row:row + n] = entry.slot
            tok_pos[row:row + n] = np.arange(pos0[index], pos0[index] + n, dtype=np.int32)
            places = [n - 1] if entry.want is None else entry.want
            want_rows.extend(row + int(p) for p in places)
            row += n
            seq_start[index + 1] = row
        self.cache.grow(growth)
        try:
            return self._run_prompts(entries, counts, pos0, total, want_rows, [
                ids, tok_slot, tok_pos,
                np.asarray([e.slot for e in entries], dtype=np.int32), seq_start,
                np.asarray(pos0, dtype=np.int32), np.asarray(want_rows, dtype=np.int32),
            ])
        except BaseException:
            # A step that could not be launched (a kernel refused a size, a part raised) leaves the sequences
            # as long as they were: the pages it took go back.  What it wrote into pages it keeps lies beyond
            # the lengths and is never read.  (Fixed-size state that a part had already advanced stays advanced.)
            self.cache.roll_back(dict(zip((e.slot for e in entries), pos0)))
            raise

    def _run_prompts(self, entries, counts, pos0, total, want_rows, arrays) -> torch.Tensor:
        longest = max(p + n for p, n in zip(pos0, counts))
        rows = prompt_rows(total)
        if (self.use_graphs and total <= PREFILL_GRAPH_MOST_TOKENS and want_rows
                and total * float(self.model.spec.width) ** 2 <= PREFILL_GRAPH_MOST_WORK):
            # a shape that comes again is replayed from a graph (engine/graph.py)
            shape = (len(counts), rows, len(want_rows), self.model.prompt_plan(len(counts), rows, longest, self.rt))
            if self._prefill_graphs is None:
                self._prefill_graphs = PrefillGraphs(self)
            done = self._prefill_graphs.step(shape, arrays, counts, pos0, longest)
            if done is not None:
                logits, self._borrowed = done
                return logits
        dev = self._stage(arrays)
        ctx = StepContext(
            tokens=total,
            batch=len(entries),
            tok_slot=dev[1],
            tok_pos=dev[2],
            seq_slot=dev[3],
            seq_start=dev[4],
            seq_pos0=dev[5],
            decode=all(n == 1 for n in counts),
            max_new=max(counts),
            max_len=longest,
            host_slots=[e.slot for e in entries],
            host_new=counts,
            host_pos0=pos0,
            plan_rows=rows,
        )
        return self.model.forward(dev[0], ctx, self.cache, dev[6], self.rt)

    def prepare_decode(self, batch: int, longest: int) -> None:
        """Makes the graph that a step of one token for each of ``batch``
        sequences replays when the longest of them has ``longest`` tokens
        after it, if it is not there yet: a caller that knows what is coming
        (a measurement, a server before it opens) pays for the capture then
        and not in the step.  Nothing of the cache changes."""
        if not self.use_graphs:
            return
        from .graph import DecodeGraphs

        if self._graphs is None:
            self._graphs = DecodeGraphs(self)
        self._graphs.get(batch, longest)

    def step_from_device(self, slots: Sequence[int], ids_device: torch.Tensor) -> torch.Tensor:
        """A step of one token per sequence whose ids are on the device already
        (int32, row j for ``slots[j]``; what a selection kernel wrote, so in
        range by construction): the host has not read them yet, and the step is
        on its way before it does.  Logits at every row, as ``step_view``
        returns them.  Only where decode steps are replayed from graphs
        (``use_graphs``)."""
        if not self.use_graphs:
            raise InvalidInput("steps from device ids need an engine that replays decode steps from graphs")
        if ids_device.dtype != torch.int32 or ids_device.dim() != 1 or ids_device.numel() < len(slots) or not slots:
            raise InvalidInput("step_from_device: one int32 id per slot is needed")
        self._borrowed = False
        self.rt.check_current()
        return self._decode_step([StepEntry(s, (), None) for s in slots], ids_device)

    def _decode_step(self, entries: Sequence[StepEntry], ids_device: Optional[torch.Tensor] = None) -> torch.Tensor:
        """A step of single tokens, replayed from a captured graph: the same
        checks as any step, without the arrays a prompt needs.  The rows
        returned view the graph's output buffer: read them before the next step."""
        from .graph import DecodeGraphs

        slots = [e.slot for e in entries]
        ids = [int(e.tokens[0]) for e in entries] if ids_device is None else None
        if len(set(slots)) != len(slots):
            twice = next(s for s in slots if slots.count(s) > 1)
            raise InvalidInput(f"slot {twice} appears twice in one step")
        if ids is not None and (min(ids) < 0 or max(ids) >= self.vocab_size):
            bad = next(t for t in ids if not 0 <= t < self.vocab_size)
            raise InvalidInput(f"token id {bad} is out of range for vocabulary {self.vocab_size}")
        for entry in entries:
            if entry.want is not None:
                for place in entry.want:
                    if int(place) != 0:
                        raise InvalidInput(f"slot {entry.slot}: wanted place {place} is not among its 1 tokens")
        if self._graphs is None:
            self._graphs = DecodeGraphs(self)
        # What only reads comes first (room in the cache, the positions' end: a step that is refused has then
        # cost no capture), then the graph (its capture may fail), the cache's growth after it: a refused
        # step changes nothing.
        checked = self.cache.check_one_more(slots)
        graph = self._graphs.get(len(entries), max(checked[0]) + 1)
        pos0 = self.cache.grow_by_one(slots, checked)
        try:
            logits = graph.run(ids, slots, pos0, ids_device)
        except BaseException:
            self.cache.roll_back(dict(zip(slots, pos0)))
            raise
        wanted = [i for i, e in enumerate(entries) if e.want is None or len(e.want) > 0]
        if len(wanted) == len(entries):
            self._borrowed = True
            return logits[: len(entries)]
        return logits[torch.tensor(wanted, dtype=torch.long, device=logits.device)]
