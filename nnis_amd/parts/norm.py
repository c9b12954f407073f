"""RMSNorm with a per-channel weight: y = x / sqrt(mean(x^2) + eps) * w
(/root/reference/crates/nnis-model/src/kernels.rs:15-48)."""

from __future__ import annotations

from .base import Norm, TensorSpec, register_part


class RMSNorm(Norm):
    graph_safe = True
    fusable_rms = True  # ``weight`` and ``eps`` are all a projection kernel needs to apply this norm itself

    def __init__(self, width: int, eps: float, weight: str):
        self.width = int(width)
        self.eps = float(eps)
        self.weight_name = weight
        self.weight = None

    def tensors(self):
        return [TensorSpec(self.weight_name, (self.width,), init="gain")]

    def bind(self, weights, rt):
        self.weight = weights[self.weight_name].contiguous()

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()

    def _out(self, x, rt, rows):
        count = x.shape[0] if rows is None else rows.shape[0]
        return rt.empty(count, self.width)

    def forward(self, x, rt, rows=None):
        return rt.ops.rmsnorm(x, self.weight, self.eps, self._out(x, rt, rows), rows=rows)

    def add_forward(self, residual, delta, rt, rows=None):
        return rt.ops.rmsnorm(residual, self.weight, self.eps, self._out(residual, rt, rows), delta=delta, rows=rows)


register_part("norm", "rms", RMSNorm)
