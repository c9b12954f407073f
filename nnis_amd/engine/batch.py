"""What one step brings: for each sequence its slot, its next tokens and the
places whose logits are wanted.  ``StepContext`` is the same on the device:
per packed token its slot and position, per sequence where it starts.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import torch


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Optional[Sequence[int]] = None  # indices into tokens; None: the last one


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
    host_new: List[int] = field(default_factory=list)
    host_pos0: List[int] = field(default_factory=list)
    splits: int = 0  # runs the keys of a decode step are cut into; 0: chosen by the kernel's wrapper
    waves: int = 1  # waves of a block of the decode attention kernel (used when splits is given)
    plan_len: int = 0  # the length each mixer plans its decode kernels for, where it is not max_len (a captured step)
    tiles: dict = field(default_factory=dict)  # work lists of prefill kernels, by tile size, made on first use
    tables: dict = field(default_factory=dict)  # the step's tables, made by the first layer that asks (``step_tables``)

    def step_tables(self, rt, rotary=None, block_table=None):
        """Each token's rows of the rotation tables ``rotary`` and its pages
        in ``block_table``, gathered once a step (``ops.StepTables``): layers
        that share a rotation and a cache group share the tables."""
        key = (None if rotary is None else rotary.cos.data_ptr(), None if block_table is None else block_table.data_ptr())
        made = self.tables.get(key)
        if made is None:
            made = self.tables[key] = rt.ops.step_tables(
                self.tok_slot, self.tok_pos, self.tokens, rotary.cos if rotary is not None else None,
                rotary.sin if rotary is not None else None, block_table, sequence_pages=self.decode)
        return made
