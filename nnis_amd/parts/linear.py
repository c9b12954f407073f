"""A projection y = W x with the checkpoint's [out, in] weight and no bias
(/root/reference/crates/nnis-model/src/runtime.rs:402-426).  The kernel is
chosen by the types at hand: 32-bit operands take the ordered 32-bit product;
bfloat16 operands take the matrix-core kernels.
"""

from __future__ import annotations

from typing import Optional

import torch


class Projection:
    def __init__(self, weight: torch.Tensor):
        if weight.dim() != 2:
            raise ValueError(f"a projection weight is a matrix, got shape {tuple(weight.shape)}")
        self.weight = weight.contiguous()
        self.out_features, self.in_features = self.weight.shape

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def __call__(self, x: torch.Tensor, rt, out_dtype: Optional[torch.dtype] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
        rows = x.shape[0]
        if out is None:
            out = rt.empty(rows, self.out_features, dtype=out_dtype or rt.dtype)
        if rows == 0:
            return out
        return rt.ops.linear(x, self.weight, out)
