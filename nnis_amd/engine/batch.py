"""What one step brings: for each sequence its slot, its next tokens and the
places whose logits are wanted.  ``StepContext`` is the same on the device:
per packed token its slot and position, per sequence where it starts.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..errors import KernelError


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Optional[Sequence[int]] = None  # indices into tokens; None: the last one


# A part's work list goes to the device through pinned memory, so that the copy does not make the host wait
# for the kernels already on the stream (a copy from ordinary memory does: 70 to 100 us a step).  One buffer
# per device, grown when a step needs more; the event says when the last copy has left it.
_list_staging: Dict[tuple, tuple] = {}


def _upload(array: np.ndarray, device) -> torch.Tensor:
    device = torch.device(device)
    count = int(array.size)
    if count == 0 or device.type != "cuda":
        return torch.from_numpy(np.ascontiguousarray(array, dtype=np.int32)).to(device)
    key = (device.type, device.index)
    held = _list_staging.get(key)
    if held is None or held[0].numel() < count:
        size = max(512, 1 << (count - 1).bit_length())
        held = _list_staging[key] = (torch.empty(size, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
    else:
        held[1].synchronize()
    host, copied = held
    host.numpy()[:count] = array.reshape(-1)
    out = torch.empty(array.shape, dtype=torch.int32, device=device)
    out.view(-1).copy_(host[:count], non_blocking=True)
    copied.record()
    return out


# what a part hands over to have a list made: (tokens each sequence brings, each sequence's first position,
# padded) -> int32 array.  ``padded`` is None for a step that is launched as it is, or (sequences, rows) of the
# fixed buffers a replayed step runs from: the array then has the size that any step of that shape can need,
# filled up with items that do nothing.  It depends on nothing else of the step.
ListMaker = Callable[[Sequence[int], Sequence[int], Optional[Tuple[int, int]]], np.ndarray]


class StepLists:
    """Work lists that parts make on the host for a step of prompts (which
    rows a block of a kernel takes, in which order), by a key of the part's
    own choosing; parts that make the same list under the same key share it.
    A step that is launched as it is makes each list on first use and copies
    it to the device."""

    def __init__(self, counts: Optional[Sequence[int]], first_positions: Optional[Sequence[int]], device):
        self.counts, self.first_positions, self.device = counts, first_positions, device
        self.made: Dict[object, torch.Tensor] = {}

    def device_list(self, key, make: ListMaker) -> torch.Tensor:
        have = self.made.get(key)
        if have is None:
            if self.counts is None or torch.cuda.is_current_stream_capturing():
                # (a copy recorded under capture would bring this step's list to every replay)
                raise KernelError(f"this step has no work list {key!r} and cannot make one")
            have = self.made[key] = _upload(make(self.counts, self.first_positions, None), self.device)
        return have


class RecordedLists(StepLists):
    """The lists of a step that runs from fixed buffers.  Its first run makes
    them as any step does, padded to the buffers' shape, and records who made
    what (``makers``); the buffers are then laid out for them
    (``engine/graph.py``) and every later step refills them from the same
    makers (``fixed``: key -> view of the fixed buffer)."""

    def __init__(self, counts, first_positions, device, padded: Tuple[int, int]):
        super().__init__(counts, first_positions, device)
        self.padded = padded
        self.makers: Dict[object, ListMaker] = {}
        self.shapes: Dict[object, tuple] = {}
        self.fixed: Optional[Dict[object, torch.Tensor]] = None

    def device_list(self, key, make: ListMaker) -> torch.Tensor:
        if self.fixed is not None:
            have = self.fixed.get(key)
            if have is None:
                raise KernelError(f"a step from fixed buffers has no work list {key!r}: its first run did not ask for it")
            return have
        have = self.made.get(key)
        if have is None:
            array = np.ascontiguousarray(make(self.counts, self.first_positions, self.padded), dtype=np.int32)
            self.makers[key], self.shapes[key] = make, array.shape
            have = self.made[key] = _upload(array, self.device)
        return have


@dataclass
class StepContext:
    tokens: int  # packed tokens of the step (rows of every activation)
    batch: int  # sequences of the step
    tok_slot: torch.Tensor  # int32 [tokens]; negative marks a padding row
    tok_pos: torch.Tensor  # int32 [tokens]: position of the token in its sequence
    seq_slot: torch.Tensor  # int32 [batch]
    seq_start: torch.Tensor  # int32 [batch + 1]: first packed row of each sequence
    seq_pos0: torch.Tensor  # int32 [batch]: position of each sequence's first new token
    decode: bool  # every sequence brings exactly one token
    max_new: int  # most tokens any sequence brings
    max_len: int  # longest sequence after this step
    host_slots: List[int] = field(default_factory=list)
    host_new: Optional[List[int]] = field(default_factory=list)
    host_pos0: Optional[List[int]] = field(default_factory=list)
    # What the parts plan their launches for, where it is not the step itself (a captured step is replayed for
    # other lengths and fewer rows than it was captured with): the longest sequence, and the step's rows.
    plan_len: int = 0
    plan_rows: int = 0
    options: dict = field(default_factory=dict)  # launch options by part kind, for tests and tuning: {"causal_attention": {...}}
    lists: Optional[StepLists] = None  # the parts' host-made work lists (``StepLists``)
    tables: dict = field(default_factory=dict)  # the step's tables, made by the first layer that asks (``step_tables``)

    def __post_init__(self):
        if self.lists is None:
            self.lists = StepLists(self.host_new, self.host_pos0, self.tok_slot.device)

    @property
    def planned_len(self) -> int:
        return self.plan_len or self.max_len

    @property
    def planned_rows(self) -> int:
        return self.plan_rows or self.tokens

    def step_tables(self, rt, rotary=None, block_table=None):
        """Each token's rows of the rotation tables ``rotary`` and its pages
        in ``block_table``, gathered once a step (``ops.StepTables``): layers
        that share a rotation and a cache group share the tables.  The
        step's positions lie below the tables' rows and its slots' pages
        inside ``block_table``: the engine refuses a step beyond either
        before anything is launched."""
        key = (None if rotary is None else rotary.cos.data_ptr(), None if block_table is None else block_table.data_ptr())
        made = self.tables.get(key)
        if made is None:
            made = self.tables[key] = rt.ops.step_tables(
                self.tok_slot, self.tok_pos, self.tokens, rotary.cos if rotary is not None else None,
                rotary.sin if rotary is not None else None, block_table, sequence_pages=self.decode)
        return made
