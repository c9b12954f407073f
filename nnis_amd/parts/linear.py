"""A projection y = W x with the checkpoint's [out, in] weight and no bias
(/root/reference/crates/nnis-model/src/runtime.rs:402-426).  The kernel is
chosen by the types at hand: a 32-bit weight takes the ordered 32-bit product;
a bfloat16 weight is packed once, when it is bound, into the order the
matrix-core kernels read, and takes those.
"""

from __future__ import annotations

from typing import Optional

import torch


class Projection:
    def __init__(self, weight: torch.Tensor, rt=None):
        """``rt``: the runtime the projection will run under; with a bfloat16
        one, a bfloat16 weight is kept packed only (the checkpoint's order is
        dropped).  Without it the weight stays as it is and takes the ordered
        product."""
        if weight.dim() != 2:
            raise ValueError(f"a projection weight is a matrix, got shape {tuple(weight.shape)}")
        self.out_features, self.in_features = weight.shape
        self._bytes = weight.numel() * weight.element_size()
        self.packed_from = None  # (address, shape) of the tensor a packed weight was made from
        if rt is not None and rt.dtype == torch.bfloat16 and rt.ops.packs(weight):
            weight = weight.contiguous()
            self.weight = rt.ops.pack_weight(weight)
            self.packed_from = (weight.data_ptr(), tuple(weight.shape))
        else:
            self.weight = weight.contiguous()

    def weight_bytes(self) -> int:
        """The weight's own bytes: what a step has to read of it."""
        return self._bytes

    def __call__(self, x: torch.Tensor, rt, out_dtype: Optional[torch.dtype] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
        rows = x.shape[0]
        if out is None:
            out = rt.empty(rows, self.out_features, dtype=out_dtype or rt.dtype)
        if rows == 0:
            return out
        return rt.ops.linear(x, self.weight, out)
