"""Helpers for the GPU tests: a runtime, a cache for one mixer, a step context
built by hand."""

import numpy as np
import torch

from nnis_amd.cache import SequenceCache
from nnis_amd.engine.batch import StepContext
from nnis_amd.engine.runtime import Runtime


def runtime(dtype):
    return Runtime("cuda:0", dtype)


def context(cache, sequences, device="cuda:0"):
    """``sequences``: list of (slot, new token count).  Grows the cache and
    returns the step context, as the engine does."""
    pos0 = [cache.length(slot) for slot, _ in sequences]
    cache.grow({slot: count for slot, count in sequences})
    tok_slot, tok_pos, starts = [], [], [0]
    for (slot, count), start in zip(sequences, pos0):
        tok_slot += [slot] * count
        tok_pos += list(range(start, start + count))
        starts.append(starts[-1] + count)
    as_dev = lambda values: torch.tensor(values, dtype=torch.int32, device=device)  # noqa: E731
    counts = [count for _, count in sequences]
    return StepContext(
        tokens=len(tok_slot), batch=len(sequences), tok_slot=as_dev(tok_slot), tok_pos=as_dev(tok_pos),
        seq_slot=as_dev([slot for slot, _ in sequences]), seq_start=as_dev(starts), seq_pos0=as_dev(pos0),
        decode=all(c == 1 for c in counts), max_new=max(counts), max_len=max(p + c for p, c in zip(pos0, counts)),
        host_slots=[slot for slot, _ in sequences], host_new=counts, host_pos0=pos0)


def cache_for(requests, rt, max_tokens=1024, max_positions=1024, shared=None):
    return SequenceCache(list(enumerate(requests)), shared or {}, max_tokens, max_positions, rt.dtype, rt.device)


def tolerance(dtype):
    return (2e-5, 2e-5) if dtype in ("float32", torch.float32) else (2e-2, 2e-2)


def assert_close(got, want, dtype, what=""):
    atol, rtol = tolerance(dtype)
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    error = (got - want).abs()
    bound = atol + rtol * want.abs()
    assert bool((error <= bound).all()), f"{what}: max error {error.max().item():.3g} (bound {atol}+{rtol}*|x|)"
