"""Trace replay through bin/trace_run, as a user runs it: the same requests
whole, with the last 32 tokens one by one, and in batches of unequal lengths
whose shorter requests end earlier, one batch after another so that slots and
pages are used again -- in 32-bit and in bfloat16, against the plain
implementation."""

import numpy as np
import pytest
import torch

import plain_llama as P
import replay
from configs import SHAPE_CONFIGS, TINY_CONFIGS
from gpu_helpers import Bf16Yardstick, Fp32Yardstick

pytestmark = pytest.mark.gpu

# lengths on purpose: 1 (a prompt that is only its first token), around a page's edge (63..65, 128..130), odd ones
LENGTHS = [1, 7, 23, 40, 64, 65, 97, 130, 5, 63]


def _requests(vocab, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, vocab, size=n).tolist() for i, n in enumerate(LENGTHS)}


def _compare(rows, plain_logits, atol, rtol, what):
    worst = 0.0
    for (name, position), row in rows.items():
        want = plain_logits[name][position].numpy()
        error = np.abs(row - want)
        bound = atol + rtol * np.abs(want)
        if np.any(error > bound):
            index = int(np.argmax(error - bound))
            raise AssertionError(f"{what}: request {name} position {position} logit {index}: "
                                 f"got {row[index]:.6f}, plain {want[index]:.6f} (max error {error.max():.3g})")
        worst = max(worst, float(error.max()))
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_schedules_agree_with_the_plain_model(model_dirs, tmp_path, name, dtype):
    config, seed = TINY_CONFIGS[name]
    vocab = config["vocab_size"]
    requests = _requests(vocab, 100 + seed)
    plain = P.PlainLlama(model_dirs[name], torch.float32)
    plain_logits = {n: plain.logits(t) for n, t in requests.items()}
    # 32-bit: rounding of sums only.  bfloat16: measured against what bfloat16 alone does to this model's
    # logits (the plain model with its activations rounded where the engine keeps them so).
    yard = Bf16Yardstick(plain, requests.values()) if dtype == "bfloat16" else None

    # every schedule in one process, one after another, with a cache too small
    # to hold them side by side: 8 pages, the largest batch needs 7
    steps = replay.whole(requests) + replay.tail_one_by_one(requests) + replay.unequal_batches(requests, batch=4, decode=32)
    count_whole = len(replay.whole(requests))
    count_tail = len(replay.tail_one_by_one(requests))
    renamed = []
    for number, step in enumerate(steps):  # one name space per schedule
        tag = "w" if number < count_whole else ("t" if number < count_whole + count_tail else "b")
        renamed.append({"entries": [dict(e, id=tag + e["id"]) for e in step["entries"]], "end": [tag + n for n in step.get("end", [])]})
    rows = replay.run_trace(model_dirs[name], dtype, renamed, str(tmp_path), max_tokens=8 * 64, vocab=vocab)
    assert len(rows) == 3 * sum(LENGTHS)
    keys = sorted((n, p) for n, t in requests.items() for p in range(len(t)))
    want = np.stack([plain_logits[n][p].numpy() for n, p in keys])
    stacked = {}
    for tag, what in (("w", "whole"), ("t", "last 32 one by one"), ("b", "unequal batches")):
        part = {(n[1:], p): row for (n, p), row in rows.items() if n[0] == tag}
        assert len(part) == sum(LENGTHS)
        if yard is None:
            _compare(part, plain_logits, 2e-5, 2e-5, f"tiny {name} {dtype} {what}")
        else:
            stacked[tag] = np.stack([part[key] for key in keys])
            yard.check(stacked[tag], want, f"tiny {name} {dtype} {what}")
    if yard is None:
        # the schedules agree with each other far more closely than with the plain model's rounding
        between = max(float(np.abs(rows[("w" + n, p)] - rows[(tag + n, p)]).max())
                      for tag in "tb" for n, t in requests.items() for p in range(len(t)))
        assert between <= 1e-5, between
    else:
        # and in bfloat16 as closely as each agrees with the plain model
        for tag in "tb":
            yard.check(stacked[tag], stacked["w"], f"tiny {name} {dtype} schedule {tag} against whole")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", sorted(SHAPE_CONFIGS))
def test_measured_shapes_agree_with_the_plain_model(tmp_path, shape, dtype):
    """The same three schedules at the layer sizes the library is measured on
    (two layers of each): wide rows, one key/value head per query head, groups
    of 8, a prompt of several pages.  32-bit: against the plain model, as for
    the tiny ones.  bfloat16: at these widths rounding alone moves a logit by
    more than the tiny models' bound, so the yardstick is the plain model run
    with its activations rounded to bfloat16 where the engine keeps them so:
    the engine may be off the 32-bit plain logits by at most 1.5 times what
    that twin is off in root mean square, and twice in the worst logit.  A
    fault (a wrong key, a mask off by one, a stale slot) moves logits by their
    own size, tens of times more."""
    import nnis_amd

    config, seed = SHAPE_CONFIGS[shape]
    folder = tmp_path / "model"
    folder.mkdir()
    nnis_amd.write_random_model(str(folder), config, seed)
    vocab = config["vocab_size"]
    rng = np.random.default_rng(seed)
    requests = {f"r{i}": rng.integers(0, vocab, size=n).tolist() for i, n in enumerate([1, 37, 65, 130, 300])}
    plain = P.PlainLlama(str(folder), torch.float32)
    plain_logits = {n: plain.logits(t) for n, t in requests.items()}
    schedules = (("w", "whole", replay.whole(requests)), ("t", "last 32 one by one", replay.tail_one_by_one(requests)),
                 ("b", "unequal batches", replay.unequal_batches(requests, batch=3, decode=32)))
    steps = []
    for tag, _, schedule in schedules:
        for step in schedule:
            steps.append({"entries": [dict(e, id=tag + e["id"]) for e in step["entries"]], "end": [tag + n for n in step.get("end", [])]})
    out = tmp_path / "out"
    out.mkdir()
    rows = replay.run_trace(str(folder), dtype, steps, str(out), max_tokens=12 * 64, vocab=vocab)
    total = sum(len(t) for t in requests.values())
    assert len(rows) == 3 * total
    if dtype == "bfloat16":
        twin = {n: plain.logits(t, P.bf16_round) for n, t in requests.items()}
        twin_error = torch.cat([(twin[n] - plain_logits[n]).flatten() for n in requests]).double()
        twin_rms, twin_worst = float(twin_error.pow(2).mean().sqrt()), float(twin_error.abs().max())
        assert 1e-4 < twin_rms < 2e-2  # the yardstick itself is rounding, not nothing and not a fault
    wide = None
    for tag, what, _ in schedules:
        part = {(n[1:], p): row for (n, p), row in rows.items() if n[0] == tag}
        assert len(part) == total
        if dtype == "float32" and config["hidden_size"] > 2048:
            # sums of up to 14,336 terms: the engine's one chain a sum against the plain model's sums in blocks
            if wide is None:
                plain64 = P.PlainLlama(str(folder), torch.float64)
                wide = Fp32Yardstick(plain64, plain, [requests["r3"], requests["r4"]])
                exact = {n: plain64.logits(t) for n, t in requests.items()}
            keys = sorted(part)
            wide.check(np.stack([part[key] for key in keys]), np.stack([exact[n][p].numpy() for n, p in keys]), f"{shape} {dtype} {what}")
            continue
        if dtype == "float32":
            _compare(part, plain_logits, 2e-5, 2e-5, f"{shape} {dtype} {what}")
            continue
        error = np.concatenate([(row - plain_logits[n][p].numpy()).ravel() for (n, p), row in part.items()]).astype(np.float64)
        rms, worst = float(np.sqrt(np.mean(error ** 2))), float(np.abs(error).max())
        assert rms <= 1.5 * twin_rms, (shape, what, rms, twin_rms)
        assert worst <= 2.0 * twin_worst, (shape, what, worst, twin_worst)
