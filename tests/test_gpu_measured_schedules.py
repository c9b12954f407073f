"""The schedules the measurements run, against the plain model: contexts of
thousands of tokens (block-table rows beyond 64 pages, keys cut into runs,
rotation rows far out), batches of 64 unequal prompts in one step with
sequences that end early and a second batch in the slots and pages of the
first, and the head's product at the real vocabularies.  Two layers of each
measured shape; the prompt's logits first, then steps fed the given next
tokens, as the reference compares
(/root/reference/crates/nnis-model/examples/compare_tiny_llama.rs:241-304).

32-bit: against the plain model in 64-bit.  bfloat16: within what bfloat16
alone does to the model's logits (``gpu_helpers.Bf16Yardstick``)."""

import numpy as np
import pytest
import torch

import plain_llama as P
from configs import SHAPE_CONFIGS
from gpu_helpers import Bf16Yardstick, Fp32Yardstick

pytestmark = pytest.mark.gpu

_MODELS = {}


def _model(tmp_path_factory, shape, max_positions):
    """(folder, plain model in 64-bit, vocabulary) of a measured shape with room for ``max_positions``."""
    import nnis_amd

    key = (shape, max_positions)
    if key not in _MODELS:
        config, seed = SHAPE_CONFIGS[shape]
        config = dict(config, max_position_embeddings=max_positions)
        folder = tmp_path_factory.mktemp(f"{shape}_{max_positions}")
        nnis_amd.write_random_model(str(folder), config, seed)
        _MODELS[key] = (str(folder), P.PlainLlama(str(folder), torch.float64), config["vocab_size"])
    return _MODELS[key]


def _check(got, want, dtype, yard, what):
    got, want = got.double().cpu(), want.double()
    if dtype == "float32" and yard is None:
        error = (got - want).abs()
        bound = 2e-5 + 2e-5 * want.abs()
        assert bool((error <= bound).all()), f"{what}: max error {error.max().item():.3g}"
    else:
        yard.check(got, want, what)


# (shape, positions the model has, tokens of the sequence)
LONG = [("smollm2-135m", 8192, 8100), ("smollm2-135m", 8192, 5000), ("smollm2-1.7b", 8192, 4200), ("tinyllama-1.1b", 2048, 2040)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape, positions, length", LONG)
def test_long_contexts(tmp_path_factory, shape, positions, length, dtype):
    """One sequence of thousands of tokens: the prompt in steps of 2,048 (each
    step's queries over all pages before them), then the last 32 tokens one by
    one (a decode step's keys cut into runs, replayed from a graph in
    bfloat16).  (Keys made loud far back, which random weights cannot give,
    are the kernels' own test: ``test_attention_beyond_64_pages``.)"""
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry

    folder, plain, vocab = _model(tmp_path_factory, shape, positions)
    rng = np.random.default_rng(length)
    ids = rng.integers(0, vocab, size=length).tolist()
    want = plain.logits(ids)
    yard = None
    if dtype == "bfloat16":
        yard = Bf16Yardstick(plain, [ids[:1500]])
    engine = load_engine(folder, dtype=dtype, max_tokens=((length + 63) // 64) * 64)
    slot = engine.start_sequence()
    head = length - 32
    # every 7th position of the prompt and all of its last 70: a 2,048-token step's full logits would be 25 MB each
    for start in range(0, head, 2048):
        count = min(2048, head - start)
        places = sorted(set(range(0, count, 7)) | set(range(max(0, count - 70), count)))
        rows = engine.step([StepEntry(slot, ids[start:start + count], places)])
        _check(rows, want[[start + p for p in places]], dtype, yard, f"{shape} {dtype} prompt rows from {start}")
    tail = [engine.step([StepEntry(slot, [ids[i]], [0])]) for i in range(head, length)]
    _check(torch.cat(tail), want[head:], dtype, yard, f"{shape} {dtype} last 32 of {length} one by one")
    assert engine.length(slot) == length
    engine.end_sequence(slot)
    assert engine.free_pages() == (length + 63) // 64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape, longest", [("smollm2-135m", 1024), ("tinyllama-1.1b", 1024), ("smollm2-1.7b", 256), ("llama-8b", 96)])
def test_batches_of_64_unequal_prompts(tmp_path_factory, shape, longest, dtype):
    """64 prompts of 16 to ``longest`` tokens in one step, then 4 steps of one
    token each during which 8 sequences end; then a second batch of 64 in a
    cache that cannot hold both, so that it runs in the slots and pages the
    first gave back."""
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry

    folder, plain, vocab = _model(tmp_path_factory, shape, 2048)
    rng = np.random.default_rng(longest + len(shape))
    first = [rng.integers(0, vocab, size=int(n) + 4).tolist() for n in rng.integers(16, longest + 1, size=64)]
    second = [rng.integers(0, vocab, size=int(n) + 2).tolist() for n in rng.integers(1, 130, size=64)]
    yard = Bf16Yardstick(plain, first[:3]) if dtype == "bfloat16" else None
    if dtype == "float32" and SHAPE_CONFIGS[shape][0]["hidden_size"] > 2048:
        yard = Fp32Yardstick(plain, P.PlainLlama(folder, torch.float32), first[:3])  # sums of 14,336 terms: see the yardstick
    pages = sum((len(t) + 63) // 64 for t in first)
    assert sum((len(t) + 63) // 64 for t in second) <= pages
    engine = load_engine(folder, dtype=dtype, max_tokens=pages * 64, max_slots=64)

    def run(batch, decode, ending):
        """Prompts (all but the last ``decode`` tokens) in one step, then one token each; ``ending[step]``:
        indices of the sequences that end after that decode step."""
        slots = [engine.start_sequence() for _ in batch]
        assert sorted(slots) == list(range(64))
        whole = [plain.logits(t) for t in batch]
        heads = [len(t) - decode for t in batch]
        rows = engine.step([StepEntry(s, t[:h], [h - 1]) for s, t, h in zip(slots, batch, heads)])
        _check(rows, torch.stack([w[h - 1] for w, h in zip(whole, heads)]), dtype, yard, f"{shape} {dtype} prompts of {len(batch)}")
        live = list(range(len(batch)))
        for step in range(decode):
            rows = engine.step([StepEntry(slots[i], [batch[i][heads[i] + step]], [0]) for i in live])
            _check(rows, torch.stack([whole[i][heads[i] + step] for i in live]), dtype, yard,
                   f"{shape} {dtype} decode step {step} of {len(live)} sequences")
            for i in ending.get(step, ()):
                engine.end_sequence(slots[i])
                live.remove(i)
        for i in live:
            engine.end_sequence(slots[i])

    free = engine.free_pages()
    run(first, 4, {0: [3, 40], 1: [0, 63, 17], 2: [9, 10, 11]})
    assert engine.free_pages() == free and engine.free_slots() == 64
    run(second, 2, {0: [5]})
    assert engine.free_pages() == free and engine.free_slots() == 64


@pytest.mark.parametrize("m", [1, 8, 64, 300])
@pytest.mark.parametrize("n, k", [(49152, 576), (49152, 2048), (32000, 2048), (128256, 4096)])
def test_the_head_at_real_vocabularies(m, n, k):
    """The head's product as every measured run launches it: whole-number
    operands, so a block that took another's rows or columns, or a strip of
    the packed table read from the wrong place, shows as a wrong integer."""
    from nnis_amd.kernels import ops

    torch.manual_seed(m + k)
    x = torch.randint(-3, 4, (m, k)).to(torch.bfloat16)
    w = torch.randint(-3, 4, (n, k)).to(torch.bfloat16)
    want = (x.cuda().double() @ w.cuda().double().t()).cpu()  # whole numbers: exact in any order
    packed = ops.pack_weight(w.cuda())
    for dtype in (torch.float32, torch.bfloat16):
        y = torch.full((m, n), 7.0, dtype=dtype, device="cuda")
        ops.gemm_bf16(x.cuda(), packed, y)
        if dtype == torch.float32:
            assert torch.equal(y.cpu().double(), want)
        else:
            assert torch.equal(y.cpu(), want.to(torch.bfloat16))
    # the same product on a prepared operand (the norm's second half in the kernel): the parts of the sums of
    # squares are chosen so that every row's mean square plus eps is 4 or 16, its scale 1/2 or 1/4
    parts = 3
    ss = torch.zeros(parts, m)
    eps = 2.0 ** -10
    ss[0] = torch.where(torch.arange(m) % 2 == 0, (4.0 - eps) * k, (16.0 - eps) * k) - 2.0
    ss[1], ss[2] = 1.5, 0.5
    scale = torch.where(torch.arange(m) % 2 == 0, 0.5, 0.25).double()
    y = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    ops.gemm_scaled(x.cuda(), ss.cuda(), parts, eps, packed, y, ops.EPILOGUE_STORE)
    scaled = want * scale[:, None]
    error = (y.cpu().double() - scaled).abs()
    assert bool((error <= 2.0 ** -8 * scaled.abs() + 1e-6).all()), error.max().item()  # one rounding to bfloat16, a root of 1 ulp
    # and the rows of a packed table come back as they went in (a head and an embedding that share it)
    rows = torch.tensor([0, 15, 16, n - 1, n // 2 + 7, -1, n], dtype=torch.int32)
    out = torch.full((rows.numel(), k), 5.0, device="cuda")
    ops.embed(rows.cuda(), packed, out)
    expect = torch.stack([w[r].float() if 0 <= r < n else torch.zeros(k) for r in rows.tolist()])
    assert torch.equal(out.cpu(), expect)
