"""The pre-norm arrangement of a layer:
x += mixer(norm1(x)); x += feed_forward(norm2(x))
(/root/reference/crates/nnis-model/src/runtime.rs:945-1095).

The residual stream is kept in 32-bit as a pair (x, pending): ``pending`` is a
part's output not yet added.  The sum is taken by the next norm in the same
kernel that normalises, and a mixer or feed-forward that starts with a
projection may take sum and norm into that projection's kernel
(``PendingNorm``), so the stream is read and written once per part.
"""

from __future__ import annotations

from .base import Block, build_part, register_part


class PreNormBlock(Block):
    def __init__(self, width, norm1, mixer, norm2, feed_forward, positions=None):
        self.width = int(width)
        self.norm1 = build_part("norm", norm1)
        self.mixer = build_part("mixer", mixer, positions=positions)
        self.norm2 = build_part("norm", norm2)
        self.feed_forward = build_part("feed_forward", feed_forward)
        self._parts = [self.norm1, self.mixer, self.norm2, self.feed_forward]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self._parts)

    def tensors(self):
        return [spec for part in self._parts for spec in part.tensors()]

    def bind(self, weights, rt):
        for part in self._parts:
            part.bind(weights, rt)

    def weight_bytes(self):
        return sum(part.weight_bytes() for part in self._parts)

    def cache_request(self):
        return self.mixer.cache_request()

    def forward(self, stream, ctx, view, rt):
        x, pending = stream
        normed = self.norm1.defer(x, pending, rt)
        if getattr(self.mixer, "takes_pending_norm", False):
            mixed = self.mixer.forward(normed, ctx, view, rt)
        else:
            mixed = self.mixer.forward(normed.materialize(), ctx, view, rt)
        normed = self.norm2.defer(normed.residual, mixed, rt)
        if getattr(self.feed_forward, "takes_pending_norm", False):
            out = self.feed_forward.forward(normed, ctx, rt)
        else:
            out = self.feed_forward.forward(normed.materialize(), ctx, rt)
        return normed.residual, out


register_part("block", "pre_norm", PreNormBlock)
