"""A norm that has not run yet.

A block hands its mixer or feed-forward ``PendingNorm(x, delta)`` instead of
the normalised rows.  A consumer whose first step is a projection can fold the
residual sum and the norm into that projection's kernel (``fused``); any other
consumer calls ``materialize`` and gets the rows from the norm's own kernel.
Either way ``residual`` afterwards holds x + delta, the stream the block goes
on with.
"""

from __future__ import annotations

from typing import Optional

import torch


class PendingNorm:
    def __init__(self, norm, x: torch.Tensor, delta: Optional[torch.Tensor], rt):
        self.norm = norm
        self.x = x
        self.delta = delta
        self.rt = rt
        self.residual: Optional[torch.Tensor] = None
        self.rows = x.shape[0]

    def materialize(self) -> torch.Tensor:
        if self.delta is None:
            out = self.norm.forward(self.x, self.rt)
        else:
            out = self.norm.add_forward(self.x, self.delta, self.rt)  # sums into x in place
        self.residual = self.x
        return out

    def can_fuse(self, weight: torch.Tensor) -> bool:
        """True when ``fused`` may be called with this projection weight."""
        ops = self.rt.ops
        return (
            getattr(self.norm, "fusable_rms", False)
            and self.rows <= ops.FUSED_MAX_TOKENS
            and self.x.dtype == torch.float32
            and weight.dtype == torch.bfloat16
            and self.rt.dtype == torch.bfloat16
            and (self.delta is None or self.delta.dtype == torch.bfloat16)
            and weight.shape[1] % 8 == 0
            and weight.data_ptr() % 16 == 0
        )

    def fused(self, weight: torch.Tensor, y: torch.Tensor, epilogue: int, rope=None) -> torch.Tensor:
        """y = epilogue(weight . norm(x + delta)) in one kernel."""
        x_out = None
        if self.delta is not None:
            x_out = torch.empty_like(self.x)
        self.rt.ops.gemm_fused(self.x, self.delta, x_out, self.norm.weight, self.norm.eps, weight, y, epilogue, rope)
        self.residual = self.x if x_out is None else x_out
        return y
