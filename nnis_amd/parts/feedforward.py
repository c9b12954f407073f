"""Gated feed-forward: down( act(gate x) * up x ), act = SiLU
(/root/reference/crates/nnis-model/src/runtime.rs:1054-1087;
/root/reference/crates/nnis-model/src/fused_swiglu.rs:14-28).  Gate and up are
one fused projection whose first ``inner`` output columns are the gate."""

from __future__ import annotations

import torch

from ..errors import Unsupported
from .base import FeedForward, TensorSpec, register_part
from .linear import Projection


class GatedFeedForward(FeedForward):
    graph_safe = True

    def __init__(self, width, inner, gate, up, down, activation="silu"):
        if activation != "silu":
            raise Unsupported(f"gated feed-forward activation {activation!r}; only silu is built")
        self.width, self.inner = int(width), int(inner)
        self.names = {"gate": gate, "up": up, "down": down}
        self.gate_up = None
        self.down = None

    def tensors(self):
        return [
            TensorSpec(self.names["gate"], (self.inner, self.width)),
            TensorSpec(self.names["up"], (self.inner, self.width)),
            TensorSpec(self.names["down"], (self.width, self.inner)),
        ]

    def bind(self, weights, rt):
        self.gate_up = Projection(torch.cat([weights[self.names["gate"]], weights[self.names["up"]]], dim=0), rt)
        self.down = Projection(weights[self.names["down"]], rt)

    def weight_bytes(self):
        return self.gate_up.weight_bytes() + self.down.weight_bytes()

    takes_pending_norm = True
    adds_to_residual = True

    def forward(self, x, ctx, rt, into=None):
        from .lazy import PendingNorm

        if isinstance(x, PendingNorm) and x.can_fuse(self.gate_up.weight):
            # (residual sum,) norm, both projections and the gating in one kernel
            hidden = x.fused(self.gate_up.weight, rt.empty(x.rows, self.inner), rt.ops.EPILOGUE_SILU)
        else:
            if isinstance(x, PendingNorm):
                x = x.materialize()
            gate_up = self.gate_up(x, rt)
            hidden = rt.ops.silu_mul(gate_up, rt.empty(x.shape[0], self.inner))
        if into is not None and into.can_take(hidden, self.down.weight):
            return into.take(hidden, self.down.weight)  # the down projection adds to the stream itself
        return self.down(hidden, rt)


register_part("feed_forward", "gated", GatedFeedForward)
