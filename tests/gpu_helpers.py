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


class Bf16Yardstick:
    """What bfloat16 alone does to a model's logits: the plain model run with
    its activations rounded to bfloat16 where the engine keeps them so (its
    twin), against the plain model in full precision, over sequences of the
    test's own.  The engine in bfloat16 may be off the plain logits by at most
    1.5 times the twin's error in root mean square (over sets of at least
    ``RMS_FROM`` logits) and twice its worst logit.  A fault -- a key missed,
    a mask off by one, a stale slot -- moves logits by several times that."""

    RMS_FROM = 16384

    def __init__(self, plain, sequences):
        errors = []
        for ids in sequences:
            ids = list(ids)
            errors.append((plain.logits(ids, _bf16_round) - plain.logits(ids)).flatten().double())
        error = torch.cat(errors)
        self.rms = float(error.pow(2).mean().sqrt())
        self.worst = float(error.abs().max())
        assert self.rms > 0 and self.worst < 0.25, (self.rms, self.worst)  # rounding: not nothing, and not a fault

    def check(self, got, want, what=""):
        """``got`` and ``want``: logits of the same shape (tensors or arrays)."""
        error = (torch.as_tensor(np.asarray(got)).double() - torch.as_tensor(np.asarray(want)).double()).flatten()
        worst = float(error.abs().max())
        assert worst <= 2.0 * self.worst, f"{what}: worst logit off by {worst:.3g}; the bfloat16 twin's worst is {self.worst:.3g}"
        if error.numel() >= self.RMS_FROM:
            rms = float(error.pow(2).mean().sqrt())
            assert rms <= 1.5 * self.rms, f"{what}: rms error {rms:.3g}; the bfloat16 twin's is {self.rms:.3g}"

    def margin(self) -> float:
        """How far below the plain model's best logit a token that the engine
        picks greedily may lie: both logits may move by the worst error."""
        return 4.0 * self.worst


class Fp32Yardstick:
    """What 32-bit sums alone do to a wide model's logits: the plain model in
    32-bit against the plain model in 64-bit.  The engine's 32-bit path sums
    as the reference does, one ascending chain of fused multiply-adds per
    output, where the plain model's library sums in blocks; a chain's
    rounding grows with its length, so the engine is off by more than the
    plain 32-bit model, by a factor that was measured at 2.0 for sums of up
    to 1,536 terms (width 576), 3.2 up to 8,192 (width 2,048) and 3.8 up to
    14,336 (width 4,096: worst logit 4.0e-5 against 1.0e-5, logits of 1.3 in
    root mean square).  Up to a width of 2,048 the flat bound of the other
    tests (2e-5 + 2e-5 |x|) is the tighter one and stays; beyond it the
    engine may be off by ``FACTOR`` times the 32-bit twin, in the worst logit
    and in root mean square.  A fault moves logits by their own size, four
    orders of magnitude more."""

    FACTOR = 6.0

    def __init__(self, plain64, plain32, sequences):
        error = torch.cat([(plain32.logits(list(ids)).double() - plain64.logits(list(ids)).double()).flatten() for ids in sequences])
        self.rms, self.worst = float(error.pow(2).mean().sqrt()), float(error.abs().max())
        assert 0 < self.worst < 1e-4, self.worst

    def check(self, got, want, what=""):
        error = (torch.as_tensor(np.asarray(got)).double() - torch.as_tensor(np.asarray(want)).double()).flatten()
        worst, rms = float(error.abs().max()), float(error.pow(2).mean().sqrt())
        assert worst <= self.FACTOR * self.worst, f"{what}: worst logit off by {worst:.3g}; the 32-bit twin's worst is {self.worst:.3g}"
        assert rms <= self.FACTOR * self.rms, f"{what}: rms error {rms:.3g}; the 32-bit twin's is {self.rms:.3g}"


def _bf16_round(x):
    return x.to(torch.bfloat16).to(x.dtype)


def tolerance(dtype):
    return (2e-5, 2e-5) if dtype in ("float32", torch.float32) else (2e-2, 2e-2)


def assert_close(got, want, dtype, what=""):
    """32-bit: rounding of sums.  bfloat16: 2e-2 of a value plus an absolute
    part that follows the size of the values compared (4e-2 of their root
    mean square, at most 2e-2): logits of a tiny model are far smaller than 1,
    and a flat bound would let a fault of their own size pass."""
    atol, rtol = tolerance(dtype)
    got, want = got.detach().float().cpu(), want.detach().float().cpu()
    if atol > 1e-3 and want.numel():
        atol = min(atol, 4e-2 * float(want.double().pow(2).mean().sqrt()))
    error = (got - want).abs()
    bound = atol + rtol * want.abs()
    assert bool((error <= bound).all()), f"{what}: max error {error.max().item():.3g} (bound {atol:.3g}+{rtol}*|x|)"
