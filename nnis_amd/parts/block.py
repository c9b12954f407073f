"""The pre-norm arrangement of a layer:
x += mixer(norm1(x)); x += feed_forward(norm2(x))
(/root/reference/crates/nnis-model/src/runtime.rs:945-1095).

The residual stream is kept in 32-bit as a pair (x, pending): ``pending`` is a
part's output not yet added.  The sum is taken by the next norm in the same
kernel that normalises, and a mixer or feed-forward that starts with a
projection may take sum and norm into that projection's kernel
(``PendingNorm``), so the stream is read and written once per part.  A part
that ends with a projection (``adds_to_residual``) may go further and add its
output to the stream in that projection's kernel, which then also prepares
the norm that follows (``ResidualInto``); the block names that norm -- its own
second one, or the first of the block that comes next (``following``).
"""

from __future__ import annotations

from .base import Block, build_part, register_part
from .lazy import PendingNorm, ResidualInto


def _joined(plans):
    """The parts' plans as one: None where none of them plans anything, the
    plan itself where one part does (the mixer, as a rule)."""
    plans = tuple(plan for plan in plans if plan is not None)
    return None if not plans else (plans[0] if len(plans) == 1 else plans)


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

    def check(self, rt):
        for part in self._parts:
            part.check(rt)

    def decode_plan(self, batch, longest, rt):
        return _joined(part.decode_plan(batch, longest, rt) for part in self._parts)

    def prompt_plan(self, batch, rows, longest, rt):
        return _joined(part.prompt_plan(batch, rows, longest, rt) for part in self._parts)

    def held_buffers(self, rt):
        return [buffer for part in self._parts for buffer in part.held_buffers(rt)]

    @property
    def entry_norm(self):
        """The norm a stream meets first here: a block before this one may prepare it."""
        return self.norm1

    def _run(self, part, normed, args, then, rt):
        """Runs a mixer or feed-forward on a pending norm; returns the pending
        norm ``then`` of the stream with the part's output (or, without
        ``then``, the stream and the output not yet added)."""
        given = normed if getattr(part, "takes_pending_norm", False) else normed.materialize()
        if then is not None and getattr(part, "adds_to_residual", False):
            out = part.forward(given, *args, into=ResidualInto(normed, then, rt))
        else:
            out = part.forward(given, *args)
        if isinstance(out, PendingNorm):
            return out
        if then is None:
            return normed.residual, out
        return then.defer(normed.residual, out, rt)

    def forward(self, stream, ctx, view, rt, following=None):
        """stream: (x, pending), or this block's first norm, pending, from the
        block before.  following: the next block's first norm, if that block
        takes it pending; then the return value is that pending norm, else the
        pair (x, pending)."""
        if isinstance(stream, PendingNorm):
            if stream.norm is not self.norm1:
                raise ValueError("the pending norm handed to a block is not the block's own first norm")
            normed = stream
        else:
            x, pending = stream
            normed = self.norm1.defer(x, pending, rt)
        normed = self._run(self.mixer, normed, (ctx, view, rt), self.norm2, rt)
        return self._run(self.feed_forward, normed, (ctx, rt), following, rt)


register_part("block", "pre_norm", PreNormBlock)
