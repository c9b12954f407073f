"""The generation loop above the step function.

Requests are taken in order, as many at a time as the batch limit and the
cache allow.  A batch's prompts are prefilled in one step, then every live
sequence gets one token per step; a sequence that emits a stop token or
reaches its own limit leaves the batch and gives its slot back at once; once a
batch has started no other request joins it.  Batches follow one another until
every request is served.

Conventions kept from the reference: the stop token is part of the returned
ids (/root/reference/crates/nnis-model/src/runtime.rs:885-890); prompt plus new
tokens must fit the positions the model has
(/root/reference/crates/nnis-model/src/sampling.rs:222-233); one generator per
sequence, seeded by the request
(/root/reference/crates/nnis-model/src/session_batch.rs:7-8).  One difference:
the last emitted token is not run through the model (the reference runs it to
leave the session continuation-ready, sampling.rs:246-249); nothing reads what
that step would compute.

The loop needs of an engine: ``vocab_size``, ``max_positions``,
``start_sequence() -> slot``, ``end_sequence(slot)``, ``step(entries) ->
logits`` and ``free_pages() -> int``; of a selector: ``start(slot, params)``
and ``select(logits, slots, params) -> tokens``.  Tests drive it with
stand-ins for both.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, FrozenSet, Iterable, List, Optional, Sequence

from ..cache.allocator import pages_for
from ..errors import CacheFull, InvalidInput
from ..sampling.params import SamplingParams
from .batch import StepEntry


@dataclass
class GenerationRequest:
    prompt: Sequence[int]
    max_new_tokens: int = 16  # the reference CLI's default (crates/nnis-cli/src/main.rs:22)
    stop_token_ids: Iterable[int] = ()
    sampling: Optional[SamplingParams] = None  # None: greedy
    on_token: Optional[Callable[[int, int], bool]] = None  # (request index, token) -> False to stop


@dataclass
class GenerationResult:
    tokens: List[int] = field(default_factory=list)
    finish_reason: str = ""  # "stop", "length" or "callback"
    prompt_tokens: int = 0


def _validate(request: GenerationRequest, index: int, vocab_size: int, max_positions: int) -> FrozenSet[int]:
    if len(request.prompt) == 0:
        # crates/nnis-model/src/runtime.rs:1135-1139
        raise InvalidInput(f"request {index}: the prompt is empty")
    if request.max_new_tokens <= 0:
        raise InvalidInput(f"request {index}: max_new_tokens must be positive; got {request.max_new_tokens}")
    if not all(0 <= int(t) < vocab_size for t in request.prompt):
        token = next(t for t in request.prompt if not 0 <= int(t) < vocab_size)
        raise InvalidInput(f"request {index}: token id {token} is out of range for vocabulary {vocab_size}")
    if len(request.prompt) + request.max_new_tokens > max_positions:
        raise InvalidInput(
            f"request {index}: prompt of {len(request.prompt)} tokens plus {request.max_new_tokens} new tokens "
            f"exceeds the model's {max_positions} positions"
        )
    stops = frozenset(int(t) for t in request.stop_token_ids)
    for token in stops:
        if not 0 <= token < vocab_size:
            # crates/nnis-model/src/config.rs:172-181
            raise InvalidInput(f"request {index}: stop token {token} is out of range for vocabulary {vocab_size}")
    if request.sampling is not None:
        request.sampling.validate(vocab_size)
    return stops


def plan_batches(needs: Sequence[int], free_pages: int, max_batch: int) -> List[List[int]]:
    """Cuts request indices, in order, into batches: at most ``max_batch``
    each, and the pages every member may come to hold (``needs``) fit the
    cache together."""
    batches: List[List[int]] = []
    current: List[int] = []
    used = 0
    for index, need in enumerate(needs):
        if need > free_pages:
            raise CacheFull(
                f"request {index} may hold {need} cache pages; the cache has {free_pages} "
                "(raise max_tokens or shorten the request)"
            )
        if current and (len(current) >= max_batch or used + need > free_pages):
            batches.append(current)
            current, used = [], 0
        current.append(index)
        used += need
    if current:
        batches.append(current)
    return batches


def generate(engine, requests: Sequence[GenerationRequest], selector=None, max_batch: int = 64) -> List[GenerationResult]:
    if max_batch <= 0:
        raise InvalidInput(f"max_batch must be positive; got {max_batch}")
    if selector is None:
        from ..sampling.device import DeviceSelector

        selector = DeviceSelector(engine)
    stops = [_validate(r, i, engine.vocab_size, engine.max_positions) for i, r in enumerate(requests)]
    results = [GenerationResult(prompt_tokens=len(r.prompt)) for r in requests]
    needs = [pages_for(len(r.prompt) + r.max_new_tokens - 1) for r in requests]
    limit = min(max_batch, engine.free_slots())
    if limit <= 0:
        raise CacheFull("the cache has no free slot")

    step = getattr(engine, "step_view", engine.step)  # the logits are read at once: no copy needed
    # An engine that takes a step's ids from the device, with a selector that leaves them there, runs a step
    # ahead of the host (below); any other pair runs step by step.
    ahead = getattr(engine, "use_graphs", False) and hasattr(engine, "step_from_device") and hasattr(selector, "select_start")

    def take(index: int, token: int, slot_of) -> bool:
        """Books one emitted token; returns whether the sequence goes on."""
        result = results[index]
        result.tokens.append(token)
        callback = requests[index].on_token
        keep_going = True if callback is None else callback(index, token) is not False
        if token in stops[index]:
            result.finish_reason = "stop"
        elif len(result.tokens) >= requests[index].max_new_tokens:
            result.finish_reason = "length"
        elif not keep_going:
            result.finish_reason = "callback"
        if result.finish_reason:
            engine.end_sequence(slot_of.pop(index))  # the slot is free for the next batch at once
            return False
        return True

    for batch in plan_batches(needs, engine.free_pages(), limit):
        live = list(batch)
        slot_of = {}
        try:
            for index in live:
                slot_of[index] = engine.start_sequence()
                selector.start(slot_of[index], requests[index].sampling)
            feed = {index: list(requests[index].prompt) for index in live}
            while live:
                logits = step([StepEntry(slot_of[i], feed[i], None) for i in live])
                pending = None
                if ahead:
                    pending = selector.select_start(logits, [slot_of[i] for i in live], [requests[i].sampling for i in live])
                if pending is not None:
                    _run_ahead(engine, selector, requests, results, slot_of, live, pending, take)
                    live = []
                    break
                tokens = selector.select(logits, [slot_of[i] for i in live], [requests[i].sampling for i in live])
                still = []
                for index, token in zip(live, tokens):
                    if take(index, int(token), slot_of):
                        feed[index] = [int(token)]
                        still.append(index)
                live = still
        finally:
            for slot in slot_of.values():  # only on an error: give everything back
                engine.end_sequence(slot)
    return results


def _run_ahead(engine, selector, requests, results, slot_of, rows, pending, take) -> None:
    """The decode steps of a batch, greedy or sampled, a step ahead of the
    host.  ``pending``: the selection of the tokens that come next, asked for
    but not read; its row j belongs to request ``rows[j]``.  Before the host
    reads them, the step that feeds them back is put on the stream, with their
    ids taken from the device, for every sequence that cannot end with that
    token by its length (``max_new_tokens``).  A sequence that the token then
    ends (a stop token, a callback) has run one step for nothing: that step's
    row is dropped, the sequence's slot is given back as always, and nothing it
    computed is read (the rows of a step do not depend on one another).  The
    tokens, their order and the reasons for ending are those of the loop that
    runs step by step."""
    import torch

    while rows:
        # who goes on whatever the token is: those whose count stays below their limit with it
        onward = [j for j, index in enumerate(rows)
                  if index in slot_of and len(results[index].tokens) + 1 < requests[index].max_new_tokens]
        following = None
        if onward:
            ids = pending.device
            if len(onward) != len(rows):
                ids = ids.index_select(0, torch.tensor(onward, dtype=torch.long, device=ids.device)).contiguous()
            logits = engine.step_from_device([slot_of[rows[j]] for j in onward], ids)
            following = selector.select_start(logits, [slot_of[rows[j]] for j in onward],
                                              [requests[rows[j]].sampling for j in onward])
        tokens = pending.result()
        for j, index in enumerate(rows):
            if index in slot_of:  # (else ended by an earlier token: this row ran for nothing)
                take(index, int(tokens[j]), slot_of)
        if following is None:
            return
        rows = [rows[j] for j in onward]  # the rows of `following`; those that ended are skipped when it is read
        pending = following
