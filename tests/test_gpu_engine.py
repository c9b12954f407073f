"""The engine in process: long decoding, the first tokens of a sequence, greedy
generation through the entry points, sampling on the device against the host
sampler, slot reuse, refused steps."""

import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as P
from configs import TINY_CONFIGS
from gpu_helpers import Bf16Yardstick

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_YARDS = {}


def _yard(model_dirs, name):
    """What bfloat16 alone does to the logits of tiny model ``name``, over sequences of several pages."""
    if name not in _YARDS:
        config, seed = TINY_CONFIGS[name]
        rng = np.random.default_rng(900 + seed)
        sequences = [rng.integers(0, config["vocab_size"], size=n).tolist() for n in (40, 97, 130, min(250, config["max_position_embeddings"]))]
        _YARDS[name] = Bf16Yardstick(P.PlainLlama(model_dirs[name]), sequences)
    return _YARDS[name]


def _engine(model_dirs, name, dtype, max_tokens=1024):
    from nnis_amd.api import load_engine

    return load_engine(model_dirs[name], dtype=dtype, max_tokens=max_tokens)


def _close(got, want, dtype, what, yard=None):
    """32-bit: rounding of sums.  bfloat16: within the model's yardstick (``_yard``)."""
    if dtype == "bfloat16":
        yard.check(got.float().cpu(), want.float().cpu(), what)
        return
    error = (got - want).abs()
    bound = 2e-5 + 2e-5 * want.abs()
    assert bool((error <= bound).all()), f"{what}: max error {error.max().item():.3g}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_long_decoding(model_dirs, name, dtype):
    """A short prompt, then several pages of single-token steps: every
    position's logits against the plain whole-sequence run."""
    from nnis_amd.engine.batch import StepEntry

    config, seed = TINY_CONFIGS[name]
    total = config["max_position_embeddings"] - 3
    ids = np.random.default_rng(seed).integers(0, config["vocab_size"], size=total).tolist()
    want = P.PlainLlama(model_dirs[name]).logits(ids)
    engine = _engine(model_dirs, name, dtype)
    slot = engine.start_sequence()
    rows = [engine.step([StepEntry(slot, ids[:3], [0, 1, 2])])]
    for token in ids[3:]:
        rows.append(engine.step([StepEntry(slot, [token], [0])]))
    got = torch.cat(rows).cpu()
    assert engine.length(slot) == total
    _close(got, want, dtype, f"tiny {name} {dtype} long decoding", _yard(model_dirs, name))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens(model_dirs, dtype):
    """A sequence's very first tokens, fed one at a time from an empty slot,
    next to a longer neighbour in the same batch."""
    from nnis_amd.engine.batch import StepEntry

    config, _ = TINY_CONFIGS["C"]
    rng = np.random.default_rng(9)
    short, long = rng.integers(0, config["vocab_size"], size=4).tolist(), rng.integers(0, config["vocab_size"], size=70).tolist()
    plain = P.PlainLlama(model_dirs["C"])
    engine = _engine(model_dirs, "C", dtype)
    a, b = engine.start_sequence(), engine.start_sequence()
    yard = _yard(model_dirs, "C")
    first = engine.step([StepEntry(a, short[:1], [0]), StepEntry(b, long[:67], [66])]).cpu()
    _close(first[0], plain.logits(short[:1])[0], dtype, "first token", yard)
    _close(first[1], plain.logits(long[:67])[66], dtype, "neighbour", yard)
    for i in range(1, 4):
        rows = engine.step([StepEntry(b, [long[66 + i]], [0]), StepEntry(a, [short[i]], None)]).cpu()
        _close(rows[1], plain.logits(short[:i + 1])[i], dtype, f"token {i}", yard)
        _close(rows[0], plain.logits(long[:67 + i])[66 + i], dtype, f"neighbour {i}", yard)


def test_refused_steps_change_nothing(model_dirs):
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.errors import CacheFull, InvalidInput

    engine = _engine(model_dirs, "A", "float32", max_tokens=128)
    slot = engine.start_sequence()
    engine.step([StepEntry(slot, [1, 2, 3], None)])
    for bad in ([StepEntry(slot, [], None)], [StepEntry(slot, [512], None)], [StepEntry(slot, [1], [1])],
                [StepEntry(slot, [1], None), StepEntry(slot, [2], None)], [StepEntry(7, [1], None)], []):
        with pytest.raises(InvalidInput):
            engine.step(bad)
    with pytest.raises(CacheFull):
        engine.step([StepEntry(slot, [1] * 126, None)])  # 129 tokens in a cache of 128
    other = engine.start_sequence()
    with pytest.raises(CacheFull):
        engine.step([StepEntry(other, [1] * 10, None), StepEntry(slot, [1] * 70, None)])  # 1 + 2 pages of 2
    assert engine.length(slot) == 3 and engine.length(other) == 0 and engine.free_pages() == 1
    with pytest.raises(CacheFull, match="positions"):
        big = _engine(model_dirs, "A", "float32", max_tokens=1024)
        s = big.start_sequence()
        big.step([StepEntry(s, [1] * 257, None)])  # the model has 256 positions


def test_a_size_the_kernels_refuse_is_refused_at_load(tmp_path):
    """A head size that the attention kernels do not take: said when the
    model is put together, before a weight is read (the folder holds none)
    or a cache made (session_batch.rs:86-101: fails before any session is
    touched)."""
    import json

    from configs import llama
    from nnis_amd.api import load_engine
    from nnis_amd.errors import Unsupported

    config = llama(num_hidden_layers=1, hidden_size=64, num_attention_heads=2, num_key_value_heads=1, head_dim=258,
                   intermediate_size=96, vocab_size=100, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
                   max_position_embeddings=128, torch_dtype="bfloat16")
    folder = tmp_path / "model"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(config))
    for dtype in ("bfloat16", "float32"):
        with pytest.raises(Unsupported, match="head_dim up to 256, got 258"):
            load_engine(str(folder), dtype=dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_that_fails_in_flight_gives_back_what_it_took(model_dirs, dtype):
    """A kernel that refuses in the middle of a step (here: the second
    layer's mixer raises) after the cache has grown: lengths and pages are as
    before, for a step of prompts and for a step of single tokens, and the
    same step then runs and is right."""
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.errors import KernelError

    engine = _engine(model_dirs, "A", dtype, max_tokens=512)
    plain = P.PlainLlama(model_dirs["A"])
    yard = _yard(model_dirs, "A") if dtype == "bfloat16" else None
    rng = np.random.default_rng(3)
    a, b = rng.integers(0, 512, size=140).tolist(), rng.integers(0, 512, size=30).tolist()
    sa, sb = engine.start_sequence(), engine.start_sequence()
    engine.step([StepEntry(sa, a[:60], None)])
    mixer = engine.model.layers[1].mixer
    forward = mixer.forward
    failing = [True]

    def sometimes(*args, **more):
        if failing[0]:
            raise KernelError("refused in flight")
        return forward(*args, **more)

    mixer.forward = sometimes
    try:
        free = engine.free_pages()
        with pytest.raises(KernelError, match="in flight"):
            engine.step([StepEntry(sa, a[60:130], None), StepEntry(sb, b[:20], None)])  # two new pages and one
        assert (engine.length(sa), engine.length(sb), engine.free_pages()) == (60, 0, free)
        failing[0] = False
        rows = engine.step([StepEntry(sa, a[60:130], None), StepEntry(sb, b[:20], None)])
        _close(rows.cpu(), torch.stack([plain.logits(a)[129], plain.logits(b)[19]]), dtype, "the step again", yard)
        # single tokens: a graph that is there already replays and cannot fail; one that has to be captured can
        engine._graphs = None
        failing[0] = True
        free = engine.free_pages()
        with pytest.raises(KernelError, match="in flight"):
            engine.step([StepEntry(sa, [a[130]], None), StepEntry(sb, [b[20]], None)])
        assert (engine.length(sa), engine.length(sb), engine.free_pages()) == (130, 20, free)
        failing[0] = False
        rows = engine.step([StepEntry(sa, [a[130]], None), StepEntry(sb, [b[20]], None)])
        _close(rows.cpu(), torch.stack([plain.logits(a)[130], plain.logits(b)[20]]), dtype, "single tokens again", yard)
    finally:
        mixer.forward = forward


def test_a_sampled_sequence_goes_on_after_a_reset(model_dirs):
    """``Engine.reset`` empties the sequence, not what the sampler keeps for
    it in the slot: temperature, top-k, top-p and the generator's state stay,
    and the draws go on (a temperature of zero left behind by a reset would
    divide the logits by zero)."""
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.sampling.device import DeviceSelector
    from nnis_amd.sampling.host import HostSampler
    from nnis_amd.sampling.params import SamplingParams

    engine = _engine(model_dirs, "B", "float32")
    params = SamplingParams(seed=11, temperature=0.7, top_k=50, top_p=0.9)
    selector = DeviceSelector(engine)
    host = HostSampler(params, engine.vocab_size)
    slot = engine.start_sequence()
    selector.start(slot, params)
    for prompt in ([5, 6, 7, 8], [9, 10], [11]):  # the second and third after a reset
        logits = engine.step([StepEntry(slot, prompt, None)])
        token = selector.select(logits, [slot], [params])[0]
        assert token == host.sample(logits[0].cpu().numpy())  # the same generator, three draws on
        engine.reset(slot)
        assert engine.length(slot) == 0


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_entry_point(model_dirs, name):
    import nnis_amd

    config, seed = TINY_CONFIGS[name]
    rng = np.random.default_rng(40 + seed)
    prompts = [rng.integers(0, config["vocab_size"], size=n).tolist() for n in (5, 11, 17, 1, 66)]
    plain = P.PlainLlama(model_dirs[name])
    stops = config.get("eos_token_id", [])
    stops = [stops] if isinstance(stops, int) else stops
    want = [plain.greedy(p, 8, stops) for p in prompts]
    # a cache of 6 pages and batches of at most 3: two batches, slots used again
    got = nnis_amd.generate(model_dirs[name], prompts, max_new_tokens=8, dtype="float32", max_tokens=6 * 64, max_batch=3)
    assert got == want
    # bfloat16 may leave the 32-bit path at a near tie: every token it picks must be the plain model's best
    # continuation of what it has picked so far, or lie below the best by no more than rounding moves two logits
    margin = _yard(model_dirs, name).margin()
    got16 = nnis_amd.generate(model_dirs[name], prompts, max_new_tokens=8, dtype="bfloat16", max_tokens=6 * 64, max_batch=3)
    at_best = total = 0
    for prompt, tokens in zip(prompts, got16):
        assert 1 <= len(tokens) <= 8
        logits = plain.logits(prompt + tokens)[len(prompt) - 1:-1]
        for row, token in zip(logits, tokens):
            assert row[token].item() >= row.max().item() - margin, (token, row[token].item(), row.max().item(), margin)
            at_best += int(token == int(row.argmax()))
            total += 1
    assert at_best >= 0.8 * total, (at_best, total)  # and near ties are the exception


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_a_step_ahead_changes_nothing(model_dirs, dtype):
    """Greedy batches run a step ahead of the host (the next step takes its
    ids from the device before the host has read them).  Tokens, their order
    in the callbacks and the reasons for ending are those of the loop that runs
    step by step: with stop tokens that are met on the way, limits of 1 and 2
    tokens, a callback that ends a sequence, more requests than a batch takes,
    and every slot given back."""
    from nnis_amd.engine.generate import GenerationRequest, generate
    from nnis_amd.sampling.device import DeviceSelector

    engine = _engine(model_dirs, "A", dtype, max_tokens=8 * 64)
    assert engine.use_graphs
    config, seed = TINY_CONFIGS["A"]
    rng = np.random.default_rng(7)
    prompts = [rng.integers(0, config["vocab_size"], size=n).tolist() for n in (5, 11, 17, 1, 30, 2, 9)]
    limits = [9, 1, 2, 12, 7, 9, 5]

    class StepByStep:  # a selector without select_start: the loop waits for every token
        def __init__(self, inner):
            self.start, self.select = inner.start, inner.select

    def run(selector, stops, stop_after):
        seen = []

        def watch(index, token):
            seen.append((index, token))
            return not (index == 3 and sum(1 for i, _ in seen if i == 3) >= stop_after)

        requests = [GenerationRequest(p, max_new_tokens=n, stop_token_ids=stops[i], on_token=watch)
                    for i, (p, n) in enumerate(zip(prompts, limits))]
        free = engine.free_slots()
        out = generate(engine, requests, selector=selector, max_batch=3)
        assert engine.free_slots() == free and engine.free_pages() == 8
        return [(r.tokens, r.finish_reason) for r in out], seen

    no_stops = [[] for _ in prompts]
    plain_run, _ = run(StepByStep(DeviceSelector(engine)), no_stops, 99)
    # stop tokens that the sequences do meet: the 4th token of request 0, the 2nd of request 4, the last of 5
    stops = [[] for _ in prompts]
    stops[0], stops[4], stops[5] = [plain_run[0][0][3]], [plain_run[4][0][1]], [plain_run[5][0][-1]]
    want, want_seen = run(StepByStep(DeviceSelector(engine)), stops, 4)
    got, got_seen = run(DeviceSelector(engine), stops, 4)
    assert got == want
    assert sorted(got_seen) == sorted(want_seen)
    for index in range(len(prompts)):  # each request's tokens reach the callback in their order
        assert [t for i, t in got_seen if i == index] == got[index][0]
    reasons = [reason for _, reason in got]
    assert reasons[0] == "stop" and reasons[1] == "length" and reasons[3] == "callback" and len(got[3][0]) == 4
    assert len(got[0][0]) <= 4 and len(got[4][0]) <= 2


def test_sampled_batches_run_a_step_ahead_too(model_dirs):
    """A batch whose rows sample (each with options and a seed of its own), next to greedy rows, runs a
    step ahead of the host like a greedy one: the tokens are those of the loop that waits for every token,
    with a stop token met on the way, requests that end early and slots used again by a second batch."""
    from nnis_amd.engine.generate import GenerationRequest, generate
    from nnis_amd.sampling import SamplingParams
    from nnis_amd.sampling.device import DeviceSelector

    engine = _engine(model_dirs, "B", "bfloat16", max_tokens=16 * 64)
    assert engine.use_graphs
    config, _ = TINY_CONFIGS["B"]
    rng = np.random.default_rng(3)
    prompts = [rng.integers(0, config["vocab_size"], size=n).tolist() for n in (4, 19, 1, 33, 8)]
    sampling = [SamplingParams(seed=11, temperature=0.7), None, SamplingParams(seed=12, temperature=1.3, top_k=5),
                SamplingParams(seed=13, temperature=0.9, top_p=0.8), SamplingParams(seed=2 ** 64 - 5, temperature=1.0)]
    limits = [10, 6, 3, 10, 1]

    class StepByStep:
        def __init__(self, inner):
            self.start, self.select = inner.start, inner.select

    def run(selector, stops):
        requests = [GenerationRequest(p, max_new_tokens=n, stop_token_ids=stops[i], sampling=sampling[i])
                    for i, (p, n) in enumerate(zip(prompts, limits))]
        out = generate(engine, requests, selector=selector, max_batch=3)
        assert engine.free_slots() == engine.cache.max_slots
        return [(r.tokens, r.finish_reason) for r in out]

    none = [[] for _ in prompts]
    free = run(StepByStep(DeviceSelector(engine)), none)
    assert run(DeviceSelector(engine), none) == free
    assert [len(tokens) for tokens, _ in free] == limits
    stops = [[] for _ in prompts]
    stops[0], stops[3] = [free[0][0][4]], [free[3][0][2]]  # the 5th sampled token of request 0, the 3rd of request 3
    want = run(StepByStep(DeviceSelector(engine)), stops)
    got = run(DeviceSelector(engine), stops)
    assert got == want
    assert got[0][1] == "stop" and len(got[0][0]) <= 5 and got[3][1] == "stop" and got[1][1] == "length"


def test_selector_refuses_a_row_that_is_not_finite(model_dirs):
    from nnis_amd.errors import InvalidInput
    from nnis_amd.sampling import SamplingParams
    from nnis_amd.sampling.device import DeviceSelector

    engine = _engine(model_dirs, "A", "float32", max_tokens=4 * 64)
    selector = DeviceSelector(engine)
    slots = [engine.start_sequence(), engine.start_sequence()]
    params = [SamplingParams(seed=1), None]
    selector.start(slots[0], params[0])
    selector.start(slots[1], params[1])
    logits = torch.zeros(2, engine.vocab_size, device="cuda")
    logits[1, 5] = 3.0
    assert selector.select(logits, slots, params)[1] == 5  # the greedy row, next to a row that samples
    logits[0, 7] = float("inf")
    with pytest.raises(InvalidInput, match="row 0"):
        selector.select(logits, slots, params)
    for slot in slots:
        engine.end_sequence(slot)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_steps_whose_shape_comes_again(model_dirs, dtype):
    """The second time a step's shape comes (sequences, tokens in all rounded up to a multiple of 64, wanted
    rows, class of the longest sequence) it is captured, from the third time on replayed: with other tokens,
    other slots, other first positions (a prompt's second run of tokens), other wanted places and the tokens
    divided otherwise among the sequences each time, the logits are the plain model's; shapes beyond the
    kept few push the oldest out, and a shape that comes back is captured again."""
    from nnis_amd.engine import graph as G
    from nnis_amd.engine.batch import StepEntry

    engine = _engine(model_dirs, "B", dtype, max_tokens=64 * 64)
    assert engine.use_graphs
    config, _ = TINY_CONFIGS["B"]
    plain = P.PlainLlama(model_dirs["B"])
    rng = np.random.default_rng(17)
    vocab = config["vocab_size"]

    def run(counts, starts, wants):
        """Sequences with ``starts[i]`` tokens already in the cache (put there in one step) bring ``counts[i]``
        more; returns nothing, checks the wanted rows against the plain model."""
        tokens = [rng.integers(0, vocab, size=s + n).tolist() for s, n in zip(starts, counts)]
        slots = [engine.start_sequence() for _ in counts]
        for slot, t, s in zip(slots, tokens, starts):
            if s:
                engine.step([StepEntry(slot, t[:s], [])])
        rows = engine.step([StepEntry(slot, t[s:], want) for slot, t, s, want in zip(slots, tokens, starts, wants)]).cpu()
        at = 0
        for t, s, n, want in zip(tokens, starts, counts, wants):
            places = [n - 1] if want is None else want
            whole = plain.logits(t)
            for place in places:
                _close(rows[at], whole[s + place], dtype, f"counts {counts} starts {starts} place {place}", _yard(model_dirs, "B"))
                at += 1
        assert at == rows.shape[0]
        for slot in slots:
            engine.end_sequence(slot)

    # the same shape five times: eager, captured, replayed three times -- other slots each time (a sequence is left
    # running between the steps), first positions 0 and beyond, wanted places that differ in where but not in how many
    keeper = engine.start_sequence()
    engine.step([StepEntry(keeper, [1, 2, 3], None)])
    run([37, 5, 70], [0, 0, 0], [[0, 36], None, [69]])
    run([37, 5, 70], [0, 0, 0], [[1, 2], None, [3]])
    graphs = engine._prefill_graphs.graphs
    of_three = lambda: [key for key in graphs if key[0] == 3]  # noqa: E731  (single prompts here share a graph of their own)
    assert [key[:3] for key in of_three()] == [(3, 128, 4)]
    other = engine.start_sequence()
    engine.step([StepEntry(other, [4, 5], None)])
    run([37, 5, 70], [3, 20, 0], [[36, 0], None, [10]])
    run([37, 5, 70], [0, 9, 30], [None, [4], [0, 69]])
    engine.end_sequence(keeper)
    run([37, 5, 70], [11, 0, 1], [[5], [0, 4], None])
    assert len(of_three()) == 1
    # the same rows (128), divided otherwise and not filled: the same graph, whose last rows belong to no sequence
    run([40, 2, 70], [0, 0, 0], [[0, 39], None, [69]])
    run([30, 30, 30], [5, 0, 64], [None, [0, 29], [7]])
    run([1, 64, 1], [0, 0, 0], [[0], [0, 63], None])
    run([64, 63, 1], [0, 1, 2], [[63], [0, 62], None])
    assert len(of_three()) == 1
    # a longer first position makes the matrix-core attention plan its launch otherwise: a shape of its own
    # (the 32-bit attention launches one way whatever the lengths: the same graph)
    run([37, 5, 70], [0, 0, 100], [[0, 36], None, [69]])
    run([37, 5, 70], [0, 0, 100], [[0, 36], None, [69]])
    assert len(of_three()) == (2 if dtype == "bfloat16" else 1)
    # more shapes than are kept: the oldest goes, and comes back through a new capture
    first = of_three()[0]
    for n in range(G.PREFILL_GRAPHS_KEPT):
        for _ in range(3):
            run([3] * (n + 5), [0] * (n + 5), [None] * (n + 5))
    assert len(graphs) == G.PREFILL_GRAPHS_KEPT and first not in graphs
    for _ in range(3):
        run([37, 5, 70], [0, 0, 0], [[0, 36], None, [69]])
    assert first in graphs
    # a step that cannot run from fixed buffers (here: a part that refuses while the step is tried from them)
    # is launched as any step, this time and from then on
    run([21, 40], [0, 0], [[0, 1, 2], [3, 4, 5]])
    from nnis_amd.errors import KernelError

    mixer = engine.model.layers[0].mixer
    forward = mixer.forward

    def refusing(x, ctx, view, rt, **more):
        if ctx.host_new is None and not ctx.decode:  # (a prompt step from a graph's buffers brings no host lists)
            raise KernelError("this part wants the host's view of the step")
        return forward(x, ctx, view, rt, **more)

    mixer.forward = refusing
    try:
        kept = list(graphs)
        for _ in range(3):
            run([21, 40], [0, 0], [[0, 7, 8], [5, 6, 9]])
        (shape,) = [key for key in engine._prefill_graphs.refused if key[:3] == (2, 64, 6)]
        assert list(graphs) == kept
    finally:
        mixer.forward = forward
    engine.end_sequence(other)
    assert engine.free_slots() == engine.cache.max_slots


def test_command_line(model_dirs):
    plain = P.PlainLlama(model_dirs["B"])
    prompt = [3, 141, 59, 26, 535]
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "nnis"), "generate", "--model", model_dirs["B"],
                          "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--dtype", "float32"],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [int(t) for t in run.stdout.strip().split(",")] == plain.greedy(prompt, 6)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "nnis"), "generate-batch", "--model", model_dirs["B"],
                          "--prompt-ids", "1,2,3", "--prompt-ids", "9", "--seed", "5", "--seed", "6", "--max-new-tokens", "4",
                          "--temperature", "0.8", "--json"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    import json

    payload = json.loads(run.stdout)
    assert payload["session_count"] == 2 and [r["seed"] for r in payload["results"]] == [5, 6]
    assert all(r["ok"] and len(r["text"].split(",")) == 4 for r in payload["results"])
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "nnis"), "generate", "--model", "/nonexistent",
                          "--prompt-ids", "1"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 1 and run.stderr.startswith("nnis generate:")


def test_command_line_with_text(model_dirs, tmp_path):
    """Text in and out through a tokenizer.json in the model folder (a word-level
    one made here), and the process entry point around the command line."""
    import json
    import shutil

    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace

    folder = str(tmp_path / "with_tokenizer")
    shutil.copytree(model_dirs["B"], folder)
    vocab = {f"w{i}": i for i in range(1000)}
    tokenizer = Tokenizer(WordLevel(vocab, unk_token="w0"))
    tokenizer.pre_tokenizer = Whitespace()
    tokenizer.save(folder + "/tokenizer.json")
    plain = P.PlainLlama(folder)
    prompt = [3, 141, 59, 26]
    want = " ".join(f"w{t}" for t in plain.greedy(prompt, 5))
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "nnis"), "generate", "--model", folder, "--prompt",
                          " ".join(f"w{t}" for t in prompt), "--max-new-tokens", "5", "--dtype", "float32"],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert run.stdout.strip() == want
    result = str(tmp_path / "result.json")
    run = subprocess.run([sys.executable, "-m", "nnis_amd.process", "--model", folder, "--prompt",
                          " ".join(f"w{t}" for t in prompt), "--max-new-tokens", "5", "--dtype", "float32", "--result", result],
                         capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert run.returncode == 0, run.stderr[-2000:]
    record = json.load(open(result))
    assert record["status"] == "generated" and record["stdout"]["utf8"].strip() == want


@pytest.mark.parametrize("options", [dict(), dict(temperature=0.8), dict(top_k=40), dict(top_p=0.7),
                                     dict(temperature=1.3, top_k=200, top_p=0.95), dict(top_k=1), dict(top_p=1.0),
                                     dict(temperature=0.05, top_p=1.0)])
@pytest.mark.parametrize("vocab", [1000, 5003, 20011, 49152, 70001])
def test_device_sampling_matches_the_host_sampler(options, vocab):
    """Same logits, same seeds: the kernel picks what the reference's host
    procedure picks, draw after draw (the generator state lives per slot).
    The vocabularies take the kernel's variants: keys in registers, 8 to 128 a
    thread, and read from memory (70,001); from 5,003 on a search starts with
    sums over the whole row and goes on with the tokens near the draw."""
    from nnis_amd.kernels import ops
    from nnis_amd.sampling import HostSampler, SamplingParams

    rows, draws = 6, 40 if vocab == 1000 else 8
    rng = np.random.default_rng(3)
    logits = (rng.standard_normal((rows, vocab)) * 2.5).astype(np.float32)
    logits[0, 5] = logits[0, 900] = logits[0].max() + 0.5  # a tie at the top
    logits[1, :] = 0.25  # all equal
    logits[2, 17] = -0.0
    logits[2, 18] = 0.0
    logits[3] = np.round(logits[3] * 4) / 4  # many ties everywhere: a draw's key is shared by hundreds
    logits[4] *= 0.02  # nearly flat: the tokens near a draw stay many for most of the search
    dev = torch.from_numpy(logits).cuda()
    slots = [4, 0, 7, 2, 5, -1]  # the last row is skipped
    state = torch.zeros(8, dtype=torch.int64, device="cuda")
    seeds = [11, 2**64 - 3, 13, 14, 15, 16]
    hosts = []
    for slot, seed in zip(slots, seeds):
        if slot >= 0:
            state[slot] = seed if seed < 2**63 else seed - 2**64
        hosts.append(HostSampler(SamplingParams(seed=seed, **options), vocab))
    temperature = torch.full((rows,), options.get("temperature", 1.0), dtype=torch.float32, device="cuda")
    top_k = torch.full((rows,), options.get("top_k", 0), dtype=torch.int32, device="cuda")
    top_p = torch.full((rows,), options.get("top_p", 0.0), dtype=torch.float32, device="cuda")
    weights = torch.empty((rows, vocab), dtype=torch.float64, device="cuda")
    row_slot = torch.tensor(slots, dtype=torch.int32, device="cuda")
    for draw in range(draws):
        out = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
        ops.sample(dev, weights, row_slot, state, temperature, top_k, top_p, out)
        got = out.cpu().tolist()
        assert got[5] == -7
        for row in range(5):
            assert got[row] == hosts[row].sample(logits[row]), (draw, row, options)
    bad = dev.clone()
    bad[3, 10] = float("nan")
    out = torch.zeros(rows, dtype=torch.int32, device="cuda")
    ops.sample(bad, weights, row_slot, state, temperature, top_k, top_p, out)
    assert out[3].item() == -1 and out[0].item() >= 0


def test_sampled_generation_is_seeded_and_per_sequence(model_dirs):
    import nnis_amd
    from nnis_amd.api import load_engine
    from nnis_amd.sampling import HostSampler, SamplingParams

    config, _ = TINY_CONFIGS["B"]
    engine = load_engine(model_dirs["B"], dtype="float32", max_tokens=512)
    prompts = [[1], [7, 8, 9, 10, 11, 12, 13], list(range(100, 123)), list(range(200, 240))]
    seeds = [7, 8, 9, 10]
    got = nnis_amd.generate(engine, prompts, max_new_tokens=12, sample=True, seed=seeds, temperature=0.8)
    again = nnis_amd.generate(engine, prompts, max_new_tokens=12, sample=True, seed=seeds, temperature=0.8)
    assert got == again and all(len(t) == 12 for t in got)
    alone = nnis_amd.generate(engine, [prompts[2]], max_new_tokens=12, sample=True, seed=9, temperature=0.8)
    assert alone[0] == got[2]  # what else is in the batch does not change a sequence
    # the plain model and the host sampler, step by step
    plain = P.PlainLlama(model_dirs["B"])
    sampler = HostSampler(SamplingParams(seed=8, temperature=0.8), config["vocab_size"])
    ids = list(prompts[1])
    for token in got[1]:
        assert sampler.sample(plain.logits(ids)[-1].numpy()) == token
        ids.append(token)
    assert engine.free_slots() == engine.cache.max_slots and engine.free_pages() == engine.cache.pages


def test_a_captured_step_keeps_the_scratch_it_was_captured_with(tmp_path):
    """The split decode attention leaves its partial sums in a scratch tensor
    that the kernels' wrapper keeps per device and replaces by a larger one
    when a step needs more.  A graph captured before has the first one's
    address baked in: it must still own that memory when it is replayed, or it
    writes into whatever the allocator has handed the block to since."""
    import nnis_amd
    from configs import SHAPE_CONFIGS
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.kernels import ops

    config, seed = SHAPE_CONFIGS["tinyllama-1.1b"]  # 32 query heads on 4: a batch of 8 at 1,100 keys needs 69,632 floats
    folder = tmp_path / "model"
    folder.mkdir()
    nnis_amd.write_random_model(str(folder), config, seed)
    plain = P.PlainLlama(str(folder))
    rng = np.random.default_rng(5)
    vocab = config["vocab_size"]
    sequences = [rng.integers(0, vocab, size=1104).tolist() for _ in range(8)]
    want = [plain.logits(sequences[i]) for i in (0, 1)]
    yard = Bf16Yardstick(plain, [sequences[0][:600]])

    ops._decode_scratch.clear()  # as in a fresh process (graphs captured by earlier tests hold what they use)
    engine = load_engine(str(folder), dtype="bfloat16", max_tokens=8 * 1152)
    assert engine.use_graphs
    a = engine.start_sequence()
    engine.step([StepEntry(a, sequences[0][:1100], [])])
    row = engine.step([StepEntry(a, [sequences[0][1100]], [0])])  # captured: one sequence, its keys in 4 runs
    yard.check(row.cpu(), want[0][1100:1101], "one sequence, first step")
    small = ops.decode_scratch_held(engine.rt.device)
    assert small is not None and small.numel() == 1 << 16
    graph = next(iter(engine._graphs.graphs.values()))
    assert [held.data_ptr() for held in graph.held] == [small.data_ptr()] * len(graph.held) and graph.held

    others = [engine.start_sequence() for _ in range(7)]
    engine.step([StepEntry(s, t[:1100], []) for s, t in zip(others, sequences[1:])])
    engine.step([StepEntry(a, [sequences[0][1101]], [0])]
                + [StepEntry(s, [t[1100]], [0]) for s, t in zip(others, sequences[1:])])  # 8 sequences: a larger scratch
    large = ops.decode_scratch_held(engine.rt.device)
    assert large.numel() > small.numel() and large.data_ptr() != small.data_ptr()
    del small
    torch.cuda.synchronize()
    sentinels = [torch.full((1 << 16,), 7.0, device="cuda") for _ in range(6)]  # what would take a freed block of that size
    assert all(s.data_ptr() != graph.held[0].data_ptr() for s in sentinels)

    for slot in others[1:]:
        engine.end_sequence(slot)
    b = others[0]
    # the first graph again, for each of two sequences alone
    row_a = engine.step([StepEntry(a, [sequences[0][1102]], [0])]).cpu()
    row_b = engine.step([StepEntry(b, [sequences[1][1101]], [0])]).cpu()
    torch.cuda.synchronize()
    assert all(bool((s == 7.0).all()) for s in sentinels)
    yard.check(row_a, want[0][1102:1103], "one sequence, replayed after the scratch grew")
    yard.check(row_b, want[1][1101:1102], "another sequence through the same graph")


def test_a_tied_head_keeps_the_table_once(model_dirs):
    """In bfloat16 the head multiplies the table in the matrix cores' packed
    order; the embedding gathers its rows from that same copy, and the table
    in the checkpoint's order is let go
    (/root/reference/crates/nnis-model/src/safetensors_loader.rs:755-786: a
    tied head shares the embedding's buffer).  32-bit: one tensor for both."""
    from nnis_amd.api import load_model
    from nnis_amd.kernels.ops import PackedWeight

    model, _ = load_model(model_dirs["A"], dtype="bfloat16")
    assert isinstance(model.embedding.table, PackedWeight)
    assert model.embedding.table is model.head.projection.weight
    untied, _ = load_model(model_dirs["B"], dtype="bfloat16")  # a head of its own: the table stays as loaded
    assert isinstance(untied.embedding.table, torch.Tensor) and isinstance(untied.head.projection.weight, PackedWeight)
    wide, _ = load_model(model_dirs["A"], dtype="float32")
    assert wide.embedding.table.data_ptr() == wide.head.projection.weight.data_ptr()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_sequence_cut_back_goes_on_from_there(model_dirs, dtype):
    """``truncate`` as the reference uses it to take back tokens a step ran
    (/root/reference/crates/nnis-rt/src/kv_cache.rs:174-192): the sequence is
    shortened across a page's edge and inside a page, goes on with other
    tokens (in a prompt step and one token at a time, replayed from graphs in
    bfloat16), and its logits are those of the sequence it now is."""
    from nnis_amd.engine.batch import StepEntry

    config, seed = TINY_CONFIGS["B"]
    rng = np.random.default_rng(70 + seed)
    first = rng.integers(0, config["vocab_size"], size=200).tolist()
    plain = P.PlainLlama(model_dirs["B"])
    yard = _yard(model_dirs, "B")
    engine = _engine(model_dirs, "B", dtype, max_tokens=8 * 64)
    slot, other = engine.start_sequence(), engine.start_sequence()
    engine.step([StepEntry(slot, first[:190], []), StepEntry(other, first[:3], [])])
    for token in first[190:]:
        engine.step([StepEntry(slot, [token], [0])])
    free = engine.free_pages()
    engine.truncate(slot, 70)  # 4 pages -> 2
    assert engine.length(slot) == 70 and engine.free_pages() == free + 2 and engine.length(other) == 3
    second = first[:70] + rng.integers(0, config["vocab_size"], size=40).tolist()
    want = plain.logits(second)
    rows = engine.step([StepEntry(slot, second[70:100], list(range(30)))])
    _close(rows.cpu(), want[70:100], dtype, "continued in one step", yard)
    rows = torch.cat([engine.step([StepEntry(slot, [token], [0])]) for token in second[100:]])
    _close(rows.cpu(), want[100:], dtype, "continued one by one", yard)
    engine.truncate(slot, 100)  # inside its second page: no page moves
    third = second[:100] + [5, 6, 7]
    rows = torch.cat([engine.step([StepEntry(slot, [token], [0])]) for token in third[100:]])
    _close(rows.cpu(), plain.logits(third)[100:], dtype, "cut back inside a page", yard)
    engine.reset(slot)
    rows = engine.step([StepEntry(slot, first[:5], [4])])
    _close(rows.cpu(), plain.logits(first[:5])[4:5], dtype, "reset and used again", yard)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name, seed", [("A", 1), ("B", 2), ("C", 3), ("B", 4)])
def test_schedules_drawn_from_a_seed(model_dirs, name, seed, dtype):
    """Sequences are started, fed in pieces of a length drawn at random (whole
    prompts, a few tokens, one token; sequences that start, go on with several
    tokens and go on with one token side by side in a step), cut back, reset
    and ended in an order drawn from the seed, in a cache of ten pages, so
    that slots and pages change hands all the time.  Every wanted row is the
    plain model's row for the sequence as it then is; a step that does not
    fit is refused and leaves everything as it was."""
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.errors import CacheFull

    config, _ = TINY_CONFIGS[name]
    rng = np.random.default_rng(1000 + seed)
    plain = P.PlainLlama(model_dirs[name])
    yard = _yard(model_dirs, name) if dtype == "bfloat16" else None
    engine = _engine(model_dirs, name, dtype, max_tokens=10 * 64)
    longest = min(300, config["max_position_embeddings"])
    live = {}  # slot -> [ids, their logits, tokens fed]

    def start():
        ids = rng.integers(0, config["vocab_size"], size=int(rng.integers(1, longest + 1))).tolist()
        live[engine.start_sequence()] = [ids, plain.logits(ids), 0]

    checked = 0
    for turn in range(150):
        action = rng.random()
        if len(live) < 2 or (action < 0.15 and len(live) < 5):
            start()
            continue
        slot = int(rng.choice(sorted(live)))
        ids, want, fed = live[slot]
        if action < 0.25:
            engine.end_sequence(slot)
            del live[slot]
            continue
        if action < 0.35 and fed > 1:  # cut back: other tokens follow from there
            keep = int(rng.integers(1, fed))
            engine.truncate(slot, keep)
            room = min(40, config["max_position_embeddings"] - keep)
            ids = ids[:keep] + rng.integers(0, config["vocab_size"], size=int(rng.integers(1, room + 1))).tolist()
            live[slot] = [ids, plain.logits(ids), keep]
            continue
        if action < 0.4:
            engine.reset(slot)
            live[slot][2] = 0
            continue
        # a step of some of the live sequences that still have tokens to feed
        some = [s for s in sorted(live) if live[s][2] < len(live[s][0]) and rng.random() < 0.7]
        if not some:
            continue
        one_each = rng.random() < 0.4  # a step of single tokens (replayed from a graph), else pieces of any length
        entries, places = [], []
        for s in some:
            ids, want, fed = live[s]
            left = len(ids) - fed
            count = 1 if one_each else int(min(left, rng.choice([1, 2, 7, 64, 65, left])))
            wanted = sorted(set(rng.integers(0, count, size=int(rng.integers(0, 4))).tolist()))
            entries.append(StepEntry(s, ids[fed:fed + count], wanted))
            places.append((s, fed, count, wanted))
        lengths = {s: engine.length(s) for s in live}
        free = engine.free_pages()
        try:
            rows = engine.step(entries)
        except CacheFull:  # more pages than the cache has left: nothing has changed, and a sequence makes room
            assert {s: engine.length(s) for s in live} == lengths and engine.free_pages() == free
            victim = max(live, key=lambda s: engine.length(s))
            engine.end_sequence(victim)
            del live[victim]
            continue
        expect = [live[s][1][fed + p] for s, fed, _, wanted in places for p in wanted]
        assert rows.shape[0] == len(expect)
        if expect:
            _close(rows.cpu(), torch.stack(expect), dtype, f"tiny {name} {dtype} seed {seed} turn {turn}", yard)
            checked += len(expect)
        for s, fed, count, _ in places:
            live[s][2] = fed + count
            assert engine.length(s) == fed + count
    assert checked >= 60
    for slot in list(live):
        engine.end_sequence(slot)
    assert engine.free_pages() == 10


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_requests_drawn_from_a_seed(model_dirs, name):
    """Batches of one to eight requests with prompts, limits, stop sets and
    a batch size drawn from a seed, through the generation loop in 32-bit, in
    a cache of twelve pages: the tokens are the plain model's greedy ones (a
    stop token is kept, as the reference keeps it), and every page comes back."""
    from nnis_amd.engine.generate import GenerationRequest, generate

    config, _ = TINY_CONFIGS[name]
    plain = P.PlainLlama(model_dirs[name])
    engine = _engine(model_dirs, name, "float32", max_tokens=12 * 64)
    for trial in range(5):
        rng = np.random.default_rng(5000 + trial)
        count = int(rng.integers(1, 9))
        prompts = [rng.integers(0, config["vocab_size"], size=int(rng.integers(1, 90))).tolist() for _ in range(count)]
        limits = [int(rng.integers(1, 25)) for _ in range(count)]
        stops = [sorted(set(rng.integers(0, config["vocab_size"], size=int(rng.integers(0, 40))).tolist())) for _ in range(count)]
        want = [plain.greedy(p, n, s) for p, n, s in zip(prompts, limits, stops)]
        out = generate(engine, [GenerationRequest(p, max_new_tokens=n, stop_token_ids=s) for p, n, s in zip(prompts, limits, stops)],
                       max_batch=int(rng.integers(1, 7)))
        assert [r.tokens for r in out] == want, f"tiny {name} trial {trial}"
        assert engine.free_pages() == 12 and engine.free_slots() == engine.cache.max_slots


def test_decode_graphs_made_ahead(model_dirs):
    """``prepare_decode`` captures the graph of a coming step and changes
    nothing else: the step then replays it and gives the plain model's logits."""
    from nnis_amd.engine.batch import StepEntry

    config, seed = TINY_CONFIGS["A"]
    ids = np.random.default_rng(seed).integers(0, config["vocab_size"], size=40).tolist()
    engine = _engine(model_dirs, "A", "bfloat16", max_tokens=4 * 64)
    slot = engine.start_sequence()
    engine.step([StepEntry(slot, ids[:30], [])])
    free, length = engine.free_pages(), engine.length(slot)
    for longest in range(31, 41):
        engine.prepare_decode(1, longest)
    graphs = dict(engine._graphs.graphs)
    assert graphs and engine.free_pages() == free and engine.length(slot) == length
    rows = torch.cat([engine.step([StepEntry(slot, [token], [0])]) for token in ids[30:]])
    assert dict(engine._graphs.graphs) == graphs  # nothing was captured on the way
    _close(rows.cpu(), P.PlainLlama(model_dirs["A"]).logits(ids)[30:], "bfloat16", "steps on graphs made ahead", _yard(model_dirs, "A"))


@pytest.mark.parametrize("heads, head_dim, inner, tokens, plan", [
    (64, 16, 512, 2048, (1, 2)), (64, 16, 512, 4096, (1, 0)),  # width 1024
    (32, 64, 1024, 2048, (4, 0)), (32, 64, 1024, 4096, (1, 2))])  # width 2048: products in tiles of 128 and 256 x 128, 256 x 192
def test_long_prompts_on_many_heads(tmp_path, heads, head_dim, inner, tokens, plan):
    """A prompt whose rows x heads give the prefill attention items for all the chip's waves: each item goes to
    one wave (of two columns at half the size, of four beyond); and at a width of 2,048 its products take the
    tiles that a step of thousands of rows is given.  One layer in bfloat16, the logits at places all along
    the prompt and of eight tokens decoded after it, against the plain model with the yardstick of its
    bfloat16 twin."""
    import nnis_amd
    from configs import llama
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.kernels import ops

    config = llama(num_hidden_layers=1, hidden_size=heads * head_dim, num_attention_heads=heads, num_key_value_heads=heads,
                   intermediate_size=inner, vocab_size=300, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=True,
                   max_position_embeddings=4096 + 64, torch_dtype="bfloat16")
    assert ops.prefill_plan(tokens, tokens, heads, head_dim, heads) == plan
    folder = str(tmp_path / "model")
    os.makedirs(folder)
    nnis_amd.write_random_model(folder, config, 5)
    ids = np.random.default_rng(tokens).integers(0, config["vocab_size"], size=tokens + 8).tolist()
    engine = load_engine(folder, dtype="bfloat16", max_tokens=tokens + 128)
    slot = engine.start_sequence()
    places = list(range(0, tokens, 193)) + list(range(tokens - 33, tokens))
    got = torch.cat([engine.step([StepEntry(slot, ids[:tokens], places)])] +
                    [engine.step([StepEntry(slot, [token], [0])]) for token in ids[tokens:]]).cpu()
    plain = P.PlainLlama(folder)
    rows = places + list(range(tokens, tokens + 8))
    Bf16Yardstick(plain, [ids[:600]]).check(got, plain.logits(ids)[rows], f"a prompt of {tokens} tokens on {heads} heads")


AWKWARD = {
    # widths and an inner size that are no multiple of 8 (no 16-byte rows: the ordered product), five heads of 16
    "width 100": dict(num_hidden_layers=2, hidden_size=100, num_attention_heads=5, num_key_value_heads=5, head_dim=16, intermediate_size=130,
                      vocab_size=777, tie_word_embeddings=True),
    # seven query heads on one key/value head, an inner size below the width, a vocabulary that is odd
    "seven on one": dict(num_hidden_layers=2, hidden_size=104, num_attention_heads=7, num_key_value_heads=1, head_dim=32, intermediate_size=100,
                         vocab_size=1003, tie_word_embeddings=False),
    # a width of 36 and a vocabulary of 61: smaller than any tile
    "width 36": dict(num_hidden_layers=1, hidden_size=36, num_attention_heads=3, num_key_value_heads=3, head_dim=16, intermediate_size=52,
                     vocab_size=61, tie_word_embeddings=True),
    # a width of 16: one strip of the stream's projections, which the tiled product still gives two parts of a row's sum of squares
    "width 16": dict(num_hidden_layers=2, hidden_size=16, num_attention_heads=2, num_key_value_heads=2, head_dim=16, intermediate_size=240,
                     vocab_size=237, tie_word_embeddings=False),
    # heads of 192 channels: beyond what the decode kernel with keys on lanes takes
    "heads of 192": dict(num_hidden_layers=2, hidden_size=192, num_attention_heads=2, num_key_value_heads=1, head_dim=192, intermediate_size=264,
                         vocab_size=333, tie_word_embeddings=True),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", sorted(AWKWARD))
def test_awkward_sizes(tmp_path, case, dtype):
    """Sizes that no kernel's tiles divide: three prompts of unequal length in one step and six tokens each one by
    one, every logit against the plain model."""
    _prompts_and_tokens_agree(tmp_path, AWKWARD[case], case, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_drawn_from_a_seed(tmp_path, dtype):
    """The same at thirty configurations whose every size is drawn from a seed: one to three layers, heads of 16 to
    256 channels in groups of one to eight, widths, inner sizes and vocabularies of any number (a width below a
    strip of 16, a vocabulary of two), a head tied or of its own."""
    import random

    rng = random.Random(20)
    for number in range(30):
        head_dim = rng.choice([16, 16, 32, 32, 48, 64, 64, 80, 96, 112, 128, 192, 256])
        kv_heads = rng.choice([1, 1, 2, 3, 4])
        group = rng.choice([1, 1, 2, 3, 4, 5, 8]) if head_dim <= 128 else rng.choice([1, 2])
        sizes = dict(num_hidden_layers=rng.randint(1, 3), hidden_size=rng.choice([rng.randint(9, 300), 8 * rng.randint(2, 60), 64 * rng.randint(1, 8)]),
                     num_attention_heads=kv_heads * group, num_key_value_heads=kv_heads, head_dim=head_dim,
                     intermediate_size=rng.choice([rng.randint(4, 500), 8 * rng.randint(1, 80)]),
                     vocab_size=rng.choice([rng.randint(2, 3000), 64 * rng.randint(1, 40)]), tie_word_embeddings=rng.random() < 0.5)
        _prompts_and_tokens_agree(tmp_path / str(number), sizes, f"drawn configuration {number} {sizes}", dtype)


def _prompts_and_tokens_agree(tmp_path, sizes, case, dtype):
    import nnis_amd
    from configs import llama
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry

    config = llama(rope_theta=10000.0, rms_norm_eps=1e-5, max_position_embeddings=256, torch_dtype="bfloat16", **sizes)
    folder = str(tmp_path / "model")
    os.makedirs(folder)
    nnis_amd.write_random_model(folder, config, 3)
    plain = P.PlainLlama(folder)
    rng = np.random.default_rng(len(case))
    sequences = [rng.integers(0, config["vocab_size"], size=n + 6).tolist() for n in (70, 9, 1)]
    yard = Bf16Yardstick(plain, sequences) if dtype == "bfloat16" else None
    engine = load_engine(folder, dtype=dtype, max_tokens=8 * 64)
    slots = [engine.start_sequence() for _ in sequences]
    got = [[] for _ in sequences]
    rows = engine.step([StepEntry(slot, ids[:-6], list(range(len(ids) - 6))) for slot, ids in zip(slots, sequences)])
    at = 0
    for i, ids in enumerate(sequences):
        got[i].append(rows[at:at + len(ids) - 6])
        at += len(ids) - 6
    for step in range(6):
        rows = engine.step([StepEntry(slot, [ids[len(ids) - 6 + step]], [0]) for slot, ids in zip(slots, sequences)])
        for i in range(len(sequences)):
            got[i].append(rows[i:i + 1])
    for i, ids in enumerate(sequences):
        _close(torch.cat(got[i]).cpu(), plain.logits(ids), dtype, f"{case}, sequence {i}", yard)
