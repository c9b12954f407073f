"""Token embedding (a row copy, /root/reference/crates/nnis-kernels/src/gather.rs:17-33)
and the output head (/root/reference/crates/nnis-model/src/runtime.rs:1109-1116),
which shares the embedding table when the checkpoint has no head of its own and
the configuration ties them
(/root/reference/crates/nnis-model/src/safetensors_loader.rs:755-786)."""

from __future__ import annotations

import torch

from .base import Part, TensorSpec, register_part
from .linear import Projection


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size, width, weight):
        self.vocab_size, self.width, self.weight_name = int(vocab_size), int(width), weight
        self.table = None

    def tensors(self):
        return [TensorSpec(self.weight_name, (self.vocab_size, self.width))]

    def bind(self, weights, rt):
        self.table = weights[self.weight_name].contiguous()

    def adopt_packed(self, source, packed) -> bool:
        """A part of the model has packed the tensor at ``source`` (address,
        shape) for the matrix cores.  If that tensor is this table (a tied
        head), rows are gathered from the packed copy from now on and the
        table in the checkpoint's order is let go: the table is kept once."""
        if isinstance(self.table, torch.Tensor) and source == (self.table.data_ptr(), tuple(self.table.shape)):
            self.table = packed
            return True
        return False

    def forward(self, ids, tokens, rt):
        """ids: int32 on the device -> the 32-bit residual stream [tokens, width]."""
        return rt.ops.embed(ids, self.table, rt.empty(tokens, self.width, dtype=torch.float32))


class LinearHead(Part):
    graph_safe = True

    def __init__(self, vocab_size, width, weight, tied_to=None):
        self.vocab_size, self.width, self.weight_name, self.tied_to = int(vocab_size), int(width), weight, tied_to
        self.projection = None

    def tensors(self):
        return [TensorSpec(self.weight_name, (self.vocab_size, self.width), fallback=self.tied_to)]

    def bind(self, weights, rt):
        # a tied head is the same device tensor as the embedding table
        self.projection = Projection(weights[self.weight_name], rt)

    def packed_sources(self):
        return [(self.projection.packed_from, self.projection.weight)] if self.projection.packed_from else []

    def weight_bytes(self):
        return self.projection.weight_bytes()

    def forward(self, x, rt):
        """Logits are 32-bit whatever the storage type."""
        return self.projection(x, rt, out_dtype=torch.float32)


register_part("embedding", "table", TokenEmbedding)
register_part("head", "linear", LinearHead)
