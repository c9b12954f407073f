"""The generation loop's decisions, driven on the CPU with stand-ins for the
engine and the token selector: batches of unequal prompts, stop tokens,
sequences that end earlier, batches one after another with slots used again."""

import numpy as np
import pytest

from nnis_amd.cache.allocator import FreeList, pages_for
from nnis_amd.engine.generate import GenerationRequest, generate, plan_batches
from nnis_amd.errors import CacheFull, InvalidInput
from nnis_amd.sampling import HostSampler, SamplingParams, greedy_token

VOCAB = 50


class ToyEngine:
    """Next-token logits favour (last token + 1) mod VOCAB.  Records every step."""

    def __init__(self, slots=4, pages=8, max_positions=200):
        self.vocab_size, self.max_positions = VOCAB, max_positions
        self._slots, self._pages = FreeList(slots, "slot"), pages
        self.lengths, self.steps, self.started, self.ended = {}, [], [], []

    def free_slots(self):
        return self._slots.free

    def free_pages(self):
        return self._pages - sum(pages_for(n) for n in self.lengths.values())

    def start_sequence(self):
        slot = self._slots.take()
        self.lengths[slot] = 0
        self.started.append(slot)
        return slot

    def end_sequence(self, slot):
        self._slots.give_back(slot)
        del self.lengths[slot]
        self.ended.append(slot)

    def step(self, entries):
        self.steps.append([(e.slot, list(e.tokens)) for e in entries])
        rows = []
        for e in entries:
            assert e.slot in self.lengths
            self.lengths[e.slot] += len(e.tokens)
            row = np.zeros(VOCAB, np.float32)
            row[(e.tokens[-1] + 1) % VOCAB] = 5.0
            rows.append(row)
        return np.stack(rows)


class HostSelector:
    def __init__(self):
        self.samplers = {}

    def start(self, slot, params):
        self.samplers[slot] = None if params is None else HostSampler(params, VOCAB)

    def select(self, logits, slots, params):
        return [greedy_token(row) if self.samplers[s] is None else self.samplers[s].sample(row)
                for row, s in zip(logits, slots)]


def test_unequal_prompts_stop_tokens_and_early_ends():
    engine = ToyEngine(slots=4)
    requests = [
        GenerationRequest([1, 2, 3], max_new_tokens=6),            # ends by length
        GenerationRequest([10], max_new_tokens=9, stop_token_ids=[13]),  # 11, 12, 13 -> stop
        GenerationRequest([20, 21], max_new_tokens=2),
    ]
    results = generate(engine, requests, HostSelector())
    assert [r.tokens for r in results] == [[4, 5, 6, 7, 8, 9], [11, 12, 13], [22, 23]]
    assert [r.finish_reason for r in results] == ["length", "stop", "length"]
    # prompts went in one step; then one token each, the live set shrinking
    assert engine.steps[0] == [(0, [1, 2, 3]), (1, [10]), (2, [20, 21])]
    assert [len(s) for s in engine.steps] == [3, 3, 2, 1, 1, 1]
    assert all(len(tokens) == 1 for step in engine.steps[1:] for _, tokens in step)
    # the last emitted token is not run: 5 decode steps for 6 new tokens
    assert len(engine.steps) == 6 and engine.lengths == {} and engine.free_slots() == 4
    assert engine.ended == [2, 1, 0]  # given back as each ends, not at the batch's end


def test_batches_follow_one_another_and_reuse_slots():
    engine = ToyEngine(slots=2)
    prompts = [[5 * i] for i in range(7)]  # a prompt token never equals a generated one (at most 3 new tokens)
    requests = [GenerationRequest(prompts[i], max_new_tokens=1 + i % 3) for i in range(7)]
    results = generate(engine, requests, HostSelector())
    for i, result in enumerate(results):  # results come in request order
        assert result.tokens == [(5 * i + 1 + k) % VOCAB for k in range(1 + i % 3)]
    assert len(engine.started) == 7 and set(engine.started) == {0, 1}  # slots are used again
    # no request joins a batch that has started: prompts enter two at a time, each pair in one step
    first = {}
    for number, step in enumerate(engine.steps):
        for _, tokens in step:
            if tokens in prompts:
                first[prompts.index(tokens)] = number
                assert all(t in prompts for _, t in step)
    assert first[0] == first[1] < first[2] == first[3] < first[4] == first[5] < first[6]
    assert engine.free_slots() == 2


def test_pages_bound_a_batch():
    assert plan_batches([2, 2, 2, 1], free_pages=4, max_batch=8) == [[0, 1], [2, 3]]
    assert plan_batches([1, 1, 1], free_pages=8, max_batch=2) == [[0, 1], [2]]
    with pytest.raises(CacheFull, match="request 1"):
        plan_batches([1, 9], free_pages=8, max_batch=4)
    engine = ToyEngine(slots=4, pages=3)
    requests = [GenerationRequest(list(range(40)), max_new_tokens=30) for _ in range(3)]  # 2 pages each
    generate(engine, requests, HostSelector())
    assert [len(s) for s in engine.steps if len(s[0][1]) == 40] == [1, 1, 1]  # one at a time


def test_seeded_sampling_is_per_sequence():
    params = SamplingParams(seed=11, temperature=5.0)
    alone = generate(ToyEngine(), [GenerationRequest([3], 12, sampling=params)], HostSelector())[0].tokens
    mixed = generate(ToyEngine(), [GenerationRequest([7, 8], 5), GenerationRequest([3], 12, sampling=params),
                                   GenerationRequest([9], 3, sampling=SamplingParams(seed=12, temperature=5.0))],
                     HostSelector())
    assert mixed[1].tokens == alone  # what else is in the batch does not change a sequence's draws
    assert mixed[0].tokens == [9, 10, 11, 12, 13] and mixed[2].tokens != alone[:3]


def test_callback_can_stop_a_sequence():
    seen = []

    def on_token(index, token):
        seen.append((index, token))
        return len(seen) < 2

    result = generate(ToyEngine(), [GenerationRequest([1], 10, on_token=on_token)], HostSelector())[0]
    assert result.tokens == [2, 3] and result.finish_reason == "callback" and seen == [(0, 2), (0, 3)]


@pytest.mark.parametrize("request_, message", [
    (GenerationRequest([], 4), "empty"),
    (GenerationRequest([1], 0), "max_new_tokens"),
    (GenerationRequest([VOCAB], 4), "out of range"),
    (GenerationRequest([1] * 190, 11), "positions"),
    (GenerationRequest([1], 4, stop_token_ids=[VOCAB + 3]), "stop token"),
    (GenerationRequest([1], 4, sampling=SamplingParams(seed=1, temperature=0.0)), "temperature"),
    (GenerationRequest([1], 4, sampling=SamplingParams(seed=1, top_k=VOCAB + 1)), "top_k"),
    (GenerationRequest([1], 4, sampling=SamplingParams(seed=1, top_p=1.5)), "top_p"),
])
def test_bad_requests_fail_before_anything_runs(request_, message):
    engine = ToyEngine()
    with pytest.raises(InvalidInput, match=message):
        generate(engine, [GenerationRequest([5], 2), request_], HostSelector())
    assert engine.steps == [] and engine.started == []


def test_an_error_mid_batch_gives_slots_back():
    engine = ToyEngine()
    original = engine.step

    def failing(entries):
        if len(engine.steps) == 2:
            raise RuntimeError("boom")
        return original(entries)

    engine.step = failing
    with pytest.raises(RuntimeError):
        generate(engine, [GenerationRequest([1], 8), GenerationRequest([2], 8)], HostSelector())
    assert engine.free_slots() == 4 and engine.lengths == {}
