"""Token selection on the device for a batch of logit rows: argmax for greedy
rows, the sampling kernel for seeded rows.  Each sequence's generator state
lives in the cache's per-slot state region, so a sequence's draws do not
depend on what else is in the batch
(/root/reference/crates/nnis-model/src/session_batch.rs:7-8)."""

from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..errors import InvalidInput
from .params import SamplingParams

RNG_REGION = "sampler.rng"


class PendingTokens:
    """Tokens that a selection kernel has been asked for: on the device at
    once (in stream order), on the host when ``result`` returns."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, event):
        self.device = device
        self._host = host
        self._event = event

    def result(self) -> List[int]:
        self._event.synchronize()
        return self._host.tolist()


class DeviceSelector:
    def __init__(self, engine):
        self.engine = engine
        self.rt = engine.rt
        self.vocab_size = engine.vocab_size
        cache = engine.cache
        if RNG_REGION not in cache.state_regions:
            cache.add_state_region(RNG_REGION, (), torch.int64)
        self.rng = cache.state_regions[RNG_REGION]
        self._weights = None
        self._picked = None       # int32 on the device, reused from step to step
        self._picked_host = None  # its pinned twin: the copy back needs no staging
        self._pairs = [None, None]  # (device, pinned host, event) of select_start, used in turn
        self._turn = 0

    def _to_host(self, picked: torch.Tensor, rows: int) -> List[int]:
        if self._picked_host is None or self._picked_host.numel() < rows:
            self._picked_host = torch.empty(max(rows, 64), dtype=torch.int32, pin_memory=True)
        host = self._picked_host[:rows]
        host.copy_(picked[:rows], non_blocking=True)
        torch.cuda.current_stream().synchronize()
        return host.tolist()

    def select_start(self, logits: torch.Tensor, slots: Sequence[int], params: Sequence[Optional[SamplingParams]]):
        """Greedy rows only: the selection is put on the stream and the copy of
        the tokens to the host behind it; nothing waits.  Returns a
        ``PendingTokens`` -- the tokens on the device (for a step that starts
        before the host has read them) and ``result()``, which waits for the
        copy -- or None when a row samples (then ``select`` is the way).  Two
        results may be outstanding at a time: the third call reuses the first's
        buffers."""
        if any(p is not None for p in params):
            return None
        rows = logits.shape[0]
        self._turn ^= 1
        pair = self._pairs[self._turn]
        if pair is None or pair[0].numel() < rows:
            size = max(rows, 64)
            pair = self._pairs[self._turn] = (torch.empty(size, dtype=torch.int32, device=self.rt.device),
                                              torch.empty(size, dtype=torch.int32, pin_memory=True), torch.cuda.Event())
        device, host, event = pair
        self.rt.ops.argmax(logits, device[:rows])
        host[:rows].copy_(device[:rows], non_blocking=True)
        event.record()
        return PendingTokens(device[:rows], host[:rows], event)

    def start(self, slot: int, params: Optional[SamplingParams]) -> None:
        """Called when a sequence starts: seeds its generator."""
        if params is not None:
            params.validate(self.vocab_size)
            seed = params.seed if params.seed < (1 << 63) else params.seed - (1 << 64)
            self.rng[slot] = seed

    def select(self, logits: torch.Tensor, slots: Sequence[int], params: Sequence[Optional[SamplingParams]]) -> List[int]:
        """One token per row of ``logits`` (float32 [rows, vocab] on the device)."""
        rows = logits.shape[0]
        ops = self.rt.ops
        if self._picked is None or self._picked.numel() < rows:
            self._picked = torch.empty(max(rows, 64), dtype=torch.int32, device=self.rt.device)
        picked = self._picked[:rows]
        ops.argmax(logits, picked)
        if any(p is not None for p in params):
            row_slot = np.asarray([s if p is not None else -1 for s, p in zip(slots, params)], dtype=np.int32)
            temperature = np.asarray([p.temperature if p is not None else 1.0 for p in params], dtype=np.float32)
            top_k = np.asarray([(p.top_k or 0) if p is not None else 0 for p in params], dtype=np.int32)
            top_p = np.asarray([(p.top_p or 0.0) if p is not None else 0.0 for p in params], dtype=np.float32)
            if self._weights is None or self._weights.shape[0] < rows:
                self._weights = torch.empty((max(rows, 8), self.vocab_size), dtype=torch.float64, device=self.rt.device)
            sampled = torch.full((rows,), -3, dtype=torch.int32, device=self.rt.device)
            ops.sample(
                logits, self._weights,
                torch.from_numpy(row_slot).to(self.rt.device), self.rng,
                torch.from_numpy(temperature).to(self.rt.device), torch.from_numpy(top_k).to(self.rt.device),
                torch.from_numpy(top_p).to(self.rt.device), sampled,
            )
            sampled_host = sampled.cpu().tolist()
            picked_host = picked.cpu().tolist()
            out = []
            for row, p in enumerate(params):
                if p is None:
                    out.append(picked_host[row])
                else:
                    if sampled_host[row] < 0:
                        raise InvalidInput(f"sampling refused row {row}: a logit is not finite")
                    out.append(sampled_host[row])
            return out
        return self._to_host(picked, rows)
