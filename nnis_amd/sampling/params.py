"""Sampling options with the reference's rules
(/root/reference/crates/nnis-model/src/sampling.rs:20-81): temperature finite
and positive (there is no temperature-0 mode; greedy is a mode of its own),
top_k in 1..=vocab, top_p in (0, 1], a seed per request."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

from ..errors import InvalidInput


@dataclass(frozen=True)
class SamplingParams:
    seed: int
    temperature: float = 1.0
    top_k: Optional[int] = None
    top_p: Optional[float] = None

    def validate(self, vocab_size: int) -> None:
        if vocab_size <= 0:
            raise InvalidInput("sampling requires a non-zero vocabulary")
        if isinstance(self.seed, bool) or not isinstance(self.seed, int) or not 0 <= self.seed < (1 << 64):
            raise InvalidInput(f"sampling seed must be an unsigned 64-bit integer; got {self.seed!r}")
        t = float(self.temperature)
        if not math.isfinite(t) or t <= 0.0:
            raise InvalidInput(f"sampling temperature must be finite and positive; got {self.temperature}")
        if self.top_k is not None:
            if isinstance(self.top_k, bool) or not isinstance(self.top_k, int) or self.top_k <= 0 or self.top_k > vocab_size:
                raise InvalidInput(f"sampling top_k must be in 1..={vocab_size}; got {self.top_k}")
        if self.top_p is not None:
            p = float(self.top_p)
            if not math.isfinite(p) or p <= 0.0 or p > 1.0:
                raise InvalidInput(f"sampling top_p must be finite and in (0, 1]; got {self.top_p}")
