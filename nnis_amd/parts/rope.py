"""Rotate-half rotary position encoding.  The tables are built once on the
host in 32-bit as the reference builds them
(/root/reference/crates/nnis-model/src/runtime.rs:1166-1184):
exponent = (2*pair)/rot_dim, inv_freq = 1/theta**exponent, angle = pos*inv_freq.
``powf``, ``cos`` and ``sin`` of a 32-bit argument are evaluated in 64-bit and
rounded once, which is what a correctly rounded 32-bit routine returns.
"""

from __future__ import annotations

import torch

from ..errors import InvalidInput
from .base import PositionEncoding, RotaryTables, register_part


def rotary_tables(positions: int, rot_dim: int, theta: float):
    half = rot_dim // 2
    pair = torch.arange(half, dtype=torch.float32)
    exponent = (2.0 * pair) / torch.tensor(float(rot_dim), dtype=torch.float32)  # 32-bit quotient
    theta32 = torch.tensor(theta, dtype=torch.float32).to(torch.float64)
    power = torch.pow(theta32, exponent.to(torch.float64)).to(torch.float32)
    inv_freq = torch.tensor(1.0, dtype=torch.float32) / power
    pos = torch.arange(positions, dtype=torch.float32)[:, None]
    angle = pos * inv_freq[None, :]  # 32-bit product
    angle64 = angle.to(torch.float64)
    return torch.cos(angle64).to(torch.float32), torch.sin(angle64).to(torch.float32)


class RotaryHalf(PositionEncoding):
    graph_safe = True

    def __init__(self, rot_dim: int, theta: float, max_positions: int):
        if rot_dim <= 0 or rot_dim % 2 != 0:
            raise InvalidInput(f"rotary dimension must be even and positive; got {rot_dim}")
        self.rot_dim = int(rot_dim)
        self.theta = float(theta)
        self.max_positions = int(max_positions)
        self._tables = None

    def bind(self, weights, rt):
        cos, sin = rotary_tables(self.max_positions, self.rot_dim, self.theta)
        self._tables = RotaryTables(cos.to(rt.device).contiguous(), sin.to(rt.device).contiguous(), self.rot_dim)

    def rotary(self):
        return self._tables


register_part("position", "rotary_half", RotaryHalf)
