"""The reference's sampler on the host, step for step
(/root/reference/crates/nnis-model/src/sampling.rs:113-202).  The device
kernel is checked against it; the generation loop's CPU tests use it."""

from __future__ import annotations

from typing import Sequence

import numpy as np

from ..errors import InvalidInput
from .params import SamplingParams
from .rng import SplitMix64


def greedy_token(logits: np.ndarray) -> int:
    """First maximum = lowest id on ties
    (/root/reference/crates/nnis-kernels/src/top_k.rs:41-92)."""
    return int(np.argmax(np.asarray(logits)))


class HostSampler:
    def __init__(self, params: SamplingParams, vocab_size: int):
        params.validate(vocab_size)
        self.params = params
        self.vocab_size = vocab_size
        self.rng = SplitMix64(params.seed)

    def sample(self, logits: Sequence[float]) -> int:
        logits = np.asarray(logits, dtype=np.float32)
        if logits.shape != (self.vocab_size,):
            raise InvalidInput(f"sampling expected {self.vocab_size} logits; got {logits.shape}")
        if not np.all(np.isfinite(logits)):
            index = int(np.flatnonzero(~np.isfinite(logits))[0])
            raise InvalidInput(f"sampling logit {index} is non-finite: {logits[index]}")
        # descending by logit, ties by lower id
        order = np.lexsort((np.arange(self.vocab_size), -logits.astype(np.float64)))
        if self.params.top_k is not None:
            order = order[: self.params.top_k]
        inv_t = 1.0 / float(np.float32(self.params.temperature))
        scaled = logits[order].astype(np.float64) * inv_t
        weights = np.exp(scaled - scaled[0])
        cumulative = np.cumsum(weights)  # a running sum in order, as the reference's loop
        total = float(cumulative[-1])
        if self.params.top_p is not None:
            threshold = float(np.float32(self.params.top_p)) * total
            crossing = int(np.argmax(cumulative >= threshold)) if np.any(cumulative >= threshold) else len(order) - 1
            retained = max(crossing + 1, 1)
            order, weights = order[:retained], weights[:retained]
            cumulative = np.cumsum(weights)
            total = float(cumulative[-1])
        draw = self.rng.next_unit() * total
        hit = np.flatnonzero(draw < cumulative)
        return int(order[hit[0]]) if hit.size else int(order[-1])
