"""The cache of a model: a slot for each live sequence; per group of layers
with the same needs, paged keys and values with a block table; beside them,
fixed-size state per slot.

Layout of a key/value group (``entries`` = schedule entries that keep a cache
in this group):
    k  [entries, pages, kv_heads, head_dim / 8, 64, 8]       8 channels of a token together
    v  [entries, pages, kv_heads, head_dim / 16, 2, 4, 16, 8] 8 tokens of a channel together
    block_table [slots, max_pages_per_slot] int32, on the device
(``layout.py`` has the orders in full: they are those in which the attention
kernels read.)
The reference's cache is [layer][kv_head][capacity][head_dim] per session
(/root/reference/crates/nnis-rt/src/kv_cache.rs:1-5,98-110); pages replace the
fixed capacity so that the memory follows the tokens actually held.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch

from ..errors import CacheFull, InvalidInput
from ..parts.base import KVRequest, StateRequest
from .allocator import PAGE_TOKENS, FreeList, PageTable, pages_for
from .layout import k_page_shape, v_page_shape


@dataclass
class KVView:
    """What an attention-like mixer sees of the cache for one schedule entry."""

    k_pages: torch.Tensor  # [pages, *k_page_shape(kv_heads, head_dim)]
    v_pages: torch.Tensor  # [pages, *v_page_shape(kv_heads, head_dim)]
    block_table: torch.Tensor  # [slots, max_pages_per_slot]
    window: Optional[int]
    read_only: bool  # this run reads another entry's cache and writes nothing


@dataclass
class StateView:
    """Fixed-size state: one row per slot, zero when a sequence starts."""

    state: torch.Tensor  # [slots, *shape]
    read_only: bool


class KVGroup:
    def __init__(self, request: KVRequest, entries: List[int], pages: int, slots: int, max_positions: int,
                 dtype: torch.dtype, device):
        self.request = request
        self.entries = entries  # schedule indices, in order
        # a windowed group has storage and pages of its own; it keeps every
        # page of a sequence (the kernels mask by the window), so that a whole
        # prompt can be written before its scores are taken
        per_slot = min(pages, pages_for(max_positions))
        self.table = PageTable(pages, slots, per_slot)
        # zero at first: a page's unwritten tail is multiplied by zero weights, so it must hold numbers
        self.k = torch.zeros((len(entries), pages) + k_page_shape(request.kv_heads, request.head_dim), dtype=dtype, device=device)
        self.v = torch.zeros((len(entries), pages) + v_page_shape(request.kv_heads, request.value_head_dim), dtype=dtype, device=device)
        pinned = torch.device(device).type == "cuda"
        self.block_table_host = torch.zeros((slots, per_slot), dtype=torch.int32, pin_memory=pinned)
        self.block_table = torch.zeros((slots, per_slot), dtype=torch.int32, device=device)
        self._table_rows = self.block_table_host.numpy()  # the same memory: an entry is written without a tensor operation
        self._dirty = set()
        # The rows go to the device by copies that do not wait (``flush``); such a copy reads the pinned row when
        # the stream gets to it, which may be long after.  Whoever writes into a row again (a slot that grows,
        # or that another sequence has taken over) first waits for the last flush to have left the pinned
        # memory: otherwise an earlier step's copy would carry the new owner's pages.
        self._flushed = torch.cuda.Event() if pinned else None
        self._flush_pending = False

    def bytes_per_token(self) -> int:
        return (len(self.entries) * self.request.kv_heads * (self.request.head_dim + self.request.value_head_dim)
                * self.k.element_size())

    def grow(self, slot: int, new_length: int) -> None:
        changed = self.table.grow(slot, new_length)
        if changed:
            self._settle()
            row = self.table.rows[slot]
            self._table_rows[slot, changed[0]:changed[-1] + 1] = row[changed[0]:changed[-1] + 1]  # (the new pages follow one another)
            self._dirty.add(slot)

    def _settle(self) -> None:
        """Waits until the last flush's copies have read the pinned rows."""
        if self._flush_pending:
            self._flushed.synchronize()
            self._flush_pending = False

    def flush(self) -> None:
        """Copies the block-table rows that changed to the device."""
        if not self._dirty:
            return
        for slot in sorted(self._dirty):
            self.block_table[slot].copy_(self.block_table_host[slot], non_blocking=True)
        self._dirty.clear()
        if self._flushed is not None:
            self._flushed.record()
            self._flush_pending = True


class SequenceCache:
    """Slots, pages and state for one model on one device.

    ``max_tokens`` is the most tokens live sequences hold at any time, each
    sequence's count rounded up to a whole page."""

    def __init__(self, requests: Sequence[Tuple[int, Any]], shared: Dict[int, int], max_tokens: int, max_positions: int,
                 dtype: torch.dtype, device, max_slots: Optional[int] = None):
        """``requests``: (schedule index, KVRequest | StateRequest | None) for
        entries that keep a cache; ``shared``: schedule index -> index of the
        entry whose cache it reads."""
        if max_tokens <= 0:
            raise InvalidInput(f"max_tokens must be positive; got {max_tokens}")
        self.device = torch.device(device)
        self.dtype = dtype
        self.max_positions = max_positions
        self.pages = pages_for(max_tokens)
        self.max_slots = min(self.pages, max_slots) if max_slots else self.pages
        self.slots = FreeList(self.max_slots, "cache slot")
        self.lengths: Dict[int, int] = {}

        self.kv_groups: List[KVGroup] = []
        self.state_regions: Dict[str, torch.Tensor] = {}
        self._layer_state: List[str] = []  # regions that a mixer's StateRequest asked for
        self._views: Dict[int, Any] = {}
        grouped: Dict[KVRequest, List[int]] = {}
        for index, request in requests:
            if isinstance(request, KVRequest):
                grouped.setdefault(request, []).append(index)
            elif isinstance(request, StateRequest):
                region = self.add_state_region(f"entry{index}", request.shape, getattr(torch, request.dtype))
                self._layer_state.append(f"entry{index}")
                self._views[index] = StateView(region, read_only=False)
            elif request is not None:
                raise InvalidInput(f"schedule entry {index}: unknown cache request {request!r}")
        for request, entries in grouped.items():
            group = KVGroup(request, entries, self.pages, self.max_slots, max_positions, dtype, self.device)
            self.kv_groups.append(group)
            for position, index in enumerate(entries):
                self._views[index] = KVView(group.k[position], group.v[position], group.block_table, request.window, False)
        for index, owner in shared.items():
            view = self._views.get(owner)
            if isinstance(view, KVView):
                self._views[index] = KVView(view.k_pages, view.v_pages, view.block_table, view.window, True)
            elif isinstance(view, StateView):
                self._views[index] = StateView(view.state, True)

    # ---- state regions ----------------------------------------------------
    def add_state_region(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        if name in self.state_regions:
            raise InvalidInput(f"state region {name!r} exists already")
        region = torch.zeros((self.max_slots, *shape), dtype=dtype, device=self.device)
        self.state_regions[name] = region
        return region

    def view(self, schedule_index: int):
        return self._views.get(schedule_index)

    # ---- slots ---------------------------------------------------------------
    def acquire(self) -> int:
        slot = self.slots.take()
        self.lengths[slot] = 0
        for region in self.state_regions.values():
            region[slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        self.slots.give_back(slot)
        del self.lengths[slot]
        for group in self.kv_groups:
            group.table.release(slot)

    def length(self, slot: int) -> int:
        try:
            return self.lengths[slot]
        except KeyError:
            raise InvalidInput(f"cache slot {slot} is not held") from None

    def truncate(self, slot: int, length: int) -> None:
        """Shortens a sequence to its first ``length`` tokens: the pages beyond
        go back to their pools at once, the tokens kept stay where they are, and
        the next step appends at ``length``
        (/root/reference/crates/nnis-rt/src/kv_cache.rs:181-192: a length above
        the current one is an error and nothing changes).  What the given-up
        part of the last page kept holds is never read: the length says where
        the data ends.  Refused where the model keeps fixed-size state per
        sequence (``StateRequest``): such state has consumed the dropped
        tokens and cannot be wound back."""
        current = self.length(slot)
        if not 0 <= int(length) <= current:
            raise InvalidInput(f"slot {slot} holds {current} tokens; it cannot be truncated to {length}")
        if length == current:
            return
        if self._layer_state:
            raise InvalidInput(
                f"slot {slot}: a model that keeps fixed-size state per sequence ({', '.join(self._layer_state)}) cannot be "
                "truncated; release the slot and run the tokens again")
        for group in self.kv_groups:
            group.table.shrink(slot, int(length))
        self.lengths[slot] = int(length)

    def reset(self, slot: int) -> None:
        """The sequence as it was before its first token: no tokens, no pages,
        and the state that the model's layers keep for it zero
        (kv_cache.rs:170-172 sets the lengths to 0).  The slot stays held,
        and so does what others keep in the slot's state regions for the
        sequence (a sampler's generator state and options): the sequence goes
        on drawing where it was."""
        self.length(slot)  # raises if the slot is not held
        for group in self.kv_groups:
            group.table.shrink(slot, 0)
        self.lengths[slot] = 0
        for name in self._layer_state:
            self.state_regions[name][slot].zero_()

    def roll_back(self, lengths: Dict[int, int]) -> None:
        """Undoes a ``grow`` whose step was not launched: each slot back to
        the length it had (never longer than it is), its pages beyond that
        back to the pools.  Unlike ``truncate`` it is not refused for fixed-size
        state, which a failed step may have touched and nothing can wind back."""
        for slot, length in lengths.items():
            if slot in self.lengths and 0 <= int(length) < self.lengths[slot]:
                for group in self.kv_groups:
                    group.table.shrink(slot, int(length))
                self.lengths[slot] = int(length)

    def check_room(self, growth: Dict[int, int]) -> None:
        """Raises before anything changes if the slots cannot grow by the given
        token counts (all or nothing, as the reference's append:
        /root/reference/crates/nnis-rt/src/kv_cache.rs:223-228)."""
        # (the end of the positions holds for every model, also for one that keeps no keys at all)
        for slot, extra in growth.items():
            new_length = self.length(slot) + extra
            if new_length > self.max_positions:
                raise CacheFull(
                    f"slot {slot} would hold {new_length} tokens; the model's positions end at {self.max_positions}"
                )
        for group in self.kv_groups:
            need = 0
            for slot, extra in growth.items():
                need += group.table.pages_needed(slot, self.lengths[slot] + extra)
            if need > group.table.pool.free:
                raise CacheFull(
                    f"the cache has {group.table.pool.free} free pages of {PAGE_TOKENS} tokens; this step needs {need}"
                )

    def grow(self, growth: Dict[int, int]) -> None:
        """Reserves pages for the new tokens and advances the lengths."""
        self.check_room(growth)
        for slot, extra in growth.items():
            new_length = self.lengths[slot] + extra
            for group in self.kv_groups:
                group.grow(slot, new_length)
            self.lengths[slot] = new_length
        for group in self.kv_groups:
            group.flush()

    def _one_more(self, slots: Sequence[int]):
        """(lengths before, slots that start a new page) of one more token for each slot; raises as ``check_room``."""
        lengths = self.lengths
        try:
            before = [lengths[slot] for slot in slots]
        except KeyError as error:
            raise InvalidInput(f"cache slot {error.args[0]} is not held") from None
        crossing = {slot: 1 for slot, length in zip(slots, before) if length % PAGE_TOKENS == 0}
        if before and max(before) >= self.max_positions:
            self.check_room({slot: 1 for slot in slots})  # raises, naming the slot
        if crossing:
            self.check_room(crossing)
        return before, crossing

    def check_one_more(self, slots: Sequence[int]):
        """Raises if ``grow_by_one`` would; changes nothing.  Returns what it
        found (the lengths now, first), which ``grow_by_one`` takes as
        ``checked`` if nothing of the cache has changed in between."""
        return self._one_more(slots)

    def grow_by_one(self, slots: Sequence[int], checked=None) -> List[int]:
        """One more token for each of the slots (a decode step): returns their
        lengths before.  Only a sequence that starts a new page takes the long
        way; all or nothing as ``grow``."""
        lengths = self.lengths
        before, crossing = checked if checked is not None else self._one_more(slots)
        if crossing:
            for slot in crossing:
                for group in self.kv_groups:
                    group.grow(slot, lengths[slot] + 1)
            for group in self.kv_groups:
                group.flush()
        for slot, length in zip(slots, before):
            lengths[slot] = length + 1
        return before

    def bytes_per_token(self) -> int:
        return sum(group.bytes_per_token() for group in self.kv_groups)

    def live_tokens(self) -> int:
        return sum(self.lengths.values())
