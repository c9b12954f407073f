"""A norm that has not run yet, or has run half.

A block hands its mixer or feed-forward a ``PendingNorm`` instead of the
normalised rows.  A consumer whose first step is a projection can fold the
norm into that projection's kernel (``fused``); any other consumer calls
``materialize`` and gets the rows from the norm's own kernel.  Either way
``residual`` afterwards holds the stream the block goes on with.

It comes in two states.  *Lazy*: ``x`` and a part's output ``delta`` that is
not added yet; the consumer's kernel takes the sum, the statistics and the
gain itself (up to ``FUSED_MAX_TOKENS`` rows).  *Prepared*: the projection
that produced the part's output has already added it to the stream and left
``scaled`` = bfloat16(stream * gain) and parts of each row's sum of squares
(``ResidualInto.take``); the consumer's kernel multiplies ``scaled`` and
applies 1 / sqrt(mean + eps) to the product, for any number of rows.
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
        self.scaled: Optional[torch.Tensor] = None  # prepared state
        self.ss: Optional[torch.Tensor] = None
        self.parts = 0

    @classmethod
    def prepared(cls, norm, residual: torch.Tensor, scaled: torch.Tensor, ss: torch.Tensor, parts: int, rt) -> "PendingNorm":
        pending = cls(norm, residual, None, rt)
        pending.residual = residual
        pending.scaled, pending.ss, pending.parts = scaled, ss, parts
        return pending

    def materialize(self) -> torch.Tensor:
        if self.delta is None:
            out = self.norm.forward(self.x, self.rt)
        else:
            out = self.norm.add_forward(self.x, self.delta, self.rt)  # sums into x in place
        self.residual = self.x
        return out

    def can_fuse(self, weight) -> bool:
        """True when ``fused`` may be called with this projection weight."""
        ops = self.rt.ops
        fits = (
            getattr(self.norm, "fusable_rms", False)
            and self.x.dtype == torch.float32
            and isinstance(weight, ops.PackedWeight)
            and self.rt.dtype == torch.bfloat16
        )
        if self.scaled is not None:
            return fits
        return fits and self.rows <= ops.FUSED_MAX_TOKENS and (self.delta is None or self.delta.dtype == torch.bfloat16)

    def fused(self, weight, y: torch.Tensor, epilogue: int, rope=None) -> torch.Tensor:
        """y = epilogue(weight . norm(x + delta)) in one kernel."""
        if self.scaled is not None:
            return self.rt.ops.gemm_scaled(self.scaled, self.ss, self.parts, self.norm.eps, weight, y, epilogue, rope)
        x_out = None
        if self.delta is not None:
            x_out = torch.empty_like(self.x)
        self.rt.ops.gemm_fused(self.x, self.delta, x_out, self.norm.weight, self.norm.eps, weight, y, epilogue, rope)
        self.residual = self.x if x_out is None else x_out
        return y


class ResidualInto:
    """Where the projection that ends a mixer or feed-forward may put its
    result instead of returning it: into the residual stream that ``source``
    (the part's own input) leaves behind, with ``norm``, the norm that comes
    next, prepared in the same kernel."""

    def __init__(self, source: PendingNorm, norm, rt):
        self.source = source
        self.norm = norm
        self.rt = rt

    def can_take(self, x: torch.Tensor, weight) -> bool:
        residual = self.source.residual
        return (
            getattr(self.norm, "fusable_rms", False)
            and residual is not None
            and residual.dtype == torch.float32
            and residual.is_contiguous()
            and self.rt.dtype == torch.bfloat16
            and x.dtype == torch.bfloat16
            and isinstance(weight, self.rt.ops.PackedWeight)
            and weight.shape[0] == residual.shape[1]
        )

    def take(self, x: torch.Tensor, weight) -> PendingNorm:
        """residual += x @ weight^T; returns the next norm, prepared."""
        rt, residual = self.rt, self.source.residual
        rows, width = residual.shape
        scaled = rt.empty(rows, width)
        ss = rt.empty(rt.ops.gemm_residual_parts(rows, width), rows, dtype=torch.float32)
        parts = rt.ops.gemm_residual(x, weight, residual, self.norm.weight, scaled, ss)
        return PendingNorm.prepared(self.norm, residual, scaled, ss, parts, rt)
