"""Each part alone against its plain function; the order of layers as data (a
layer named twice, a layer that reads another layer's cache); and a toy mixer
with state of its own, defined here, registered, built and stepped without a
change to the library's files."""

import math
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import plain_llama as P
from gpu_helpers import assert_close, cache_for, context, runtime, tolerance

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def _w(shape, dtype, seed, gain=False):
    g = torch.Generator().manual_seed(seed)
    noise = torch.randn(shape, generator=g)
    value = 1.0 + 0.1 * noise if gain else noise / math.sqrt(shape[-1])
    return value.to(torch.bfloat16 if dtype == "bfloat16" else torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(dtype):
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    width, eps = 70, 3e-4
    norm = build_part("norm", {"kind": "rms", "width": width, "eps": eps, "weight": "n.w"})
    assert [(t.name, t.shape, t.init) for t in norm.tensors()] == [("n.w", (70,), "gain")]
    weight = _w((width,), dtype, 1, gain=True)
    norm.bind({"n.w": weight.cuda()}, rt)
    x = torch.randn(9, width) * 3
    delta = torch.randn(9, width).to(rt.dtype)
    assert_close(norm.forward(x.cuda(), rt), P.rms_norm(x, weight.float(), eps), dtype, "norm")
    stream = x.cuda().clone()
    got = norm.add_forward(stream, delta.cuda(), rt)
    assert_close(got, P.rms_norm(x + delta.float(), weight.float(), eps), dtype, "add + norm")
    assert torch.equal(stream.cpu(), x + delta.float())  # the residual sum is kept in 32-bit
    rows = torch.tensor([8, 0, 3], dtype=torch.int32).cuda()
    stream = x.cuda().clone()
    got = norm.add_forward(stream, delta.cuda(), rt, rows=rows)
    assert_close(got, P.rms_norm((x + delta.float())[[8, 0, 3]], weight.float(), eps), dtype, "gathered rows")
    assert torch.equal(stream.cpu(), x)  # a gather writes nothing back


def test_rotary_tables_equal_the_plain_ones():
    from nnis_amd.parts import build_part

    rt = runtime("float32")
    for rot_dim, theta, positions in ((16, 10000.0, 256), (32, 100000.0, 512), (64, 130000.0, 8192)):
        part = build_part("position", {"kind": "rotary_half", "rot_dim": rot_dim, "theta": theta, "max_positions": positions})
        part.bind({}, rt)
        tables = part.rotary()
        cos, sin = P.rope_tables(positions, rot_dim, theta)
        assert tables.rot_dim == rot_dim and tables.cos.dtype == torch.float32
        assert np.abs(tables.cos.cpu().numpy() - cos).max() <= 6e-8 and np.abs(tables.sin.cpu().numpy() - sin).max() <= 6e-8


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, head_dim, width", [(4, 2, 16, 64), (3, 1, 32, 80), (6, 6, 48, 100), (2, 1, 192, 96), (3, 3, 256, 96)])
def test_attention_part(dtype, heads, kv_heads, head_dim, width):
    """Two sequences of unequal length, whole and then continued by single
    tokens, against the plain functions on each whole sequence."""
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    rope = build_part("position", {"kind": "rotary_half", "rot_dim": head_dim, "theta": 5000.0, "max_positions": 300})
    rope.bind({}, rt)
    mixer = build_part("mixer", {"kind": "causal_attention", "width": width, "heads": heads, "kv_heads": kv_heads,
                                 "head_dim": head_dim, "position": "r", "q": "q", "k": "k", "v": "v", "o": "o"},
                       positions={"r": rope})
    shapes = {t.name: t.shape for t in mixer.tensors()}
    assert shapes == {"q": (heads * head_dim, width), "k": (kv_heads * head_dim, width),
                      "v": (kv_heads * head_dim, width), "o": (width, heads * head_dim)}
    weights = {n: _w(s, dtype, i) for i, (n, s) in enumerate(shapes.items())}
    mixer.bind({n: w.cuda() for n, w in weights.items()}, rt)
    cache = cache_for([mixer.cache_request()], rt)
    lengths = (70, 9)
    xs = [torch.randn(n + 3, width).to(rt.dtype) for n in lengths]
    cos, sin = (torch.from_numpy(t) for t in P.rope_tables(300, head_dim, 5000.0))

    def plain(x):
        t = x.shape[0]
        x = x.float()
        q = P.linear(x, weights["q"].float()).view(t, heads, head_dim)
        k = P.linear(x, weights["k"].float()).view(t, kv_heads, head_dim)
        v = P.linear(x, weights["v"].float()).view(t, kv_heads, head_dim)
        q, k = P.rope_rotate_half(q, cos[:t], sin[:t]), P.rope_rotate_half(k, cos[:t], sin[:t])
        out = P.causal_attention(q, k, v, 1.0 / math.sqrt(head_dim)).reshape(t, heads * head_dim)
        return P.linear(out, weights["o"].float())

    want = [plain(x) for x in xs]
    slots = [cache.acquire(), cache.acquire(), cache.acquire()][1:]  # not slot 0
    ctx = context(cache, list(zip(slots, lengths)))
    got = mixer.forward(torch.cat([x[:n] for x, n in zip(xs, lengths)]).cuda(), ctx, cache.view(0), rt)
    assert_close(got[:70], want[0][:70], dtype, "prompt 0")
    assert_close(got[70:], want[1][:9], dtype, "prompt 1")
    for step in range(3):
        ctx = context(cache, [(slots[1], 1), (slots[0], 1)])  # the other order
        x = torch.stack([xs[1][9 + step], xs[0][70 + step]]).cuda()
        got = mixer.forward(x, ctx, cache.view(0), rt)
        assert_close(got[0], want[1][9 + step], dtype, f"decode {step} seq 1")
        assert_close(got[1], want[0][70 + step], dtype, f"decode {step} seq 0")


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_embedding_and_head_parts(dtype):
    from nnis_amd.parts import build_part

    rt = runtime(dtype)
    width, inner, vocab = 72, 200, 333
    ff = build_part("feed_forward", {"kind": "gated", "width": width, "inner": inner, "activation": "silu",
                                     "gate": "g", "up": "u", "down": "d"})
    weights = {"g": _w((inner, width), dtype, 1), "u": _w((inner, width), dtype, 2), "d": _w((width, inner), dtype, 3)}
    ff.bind({n: w.cuda() for n, w in weights.items()}, rt)
    x = torch.randn(11, width).to(rt.dtype)
    want = P.swiglu(x.float(), weights["g"].float(), weights["u"].float(), weights["d"].float())
    assert_close(ff.forward(x.cuda(), None, rt), want, dtype, "gated feed-forward")

    table = _w((vocab, width), dtype, 4)
    emb = build_part("embedding", {"kind": "table", "vocab_size": vocab, "width": width, "weight": "e"})
    emb.bind({"e": table.cuda()}, rt)
    ids = torch.tensor([0, 332, 17, 17], dtype=torch.int32)
    got = emb.forward(ids.cuda(), 4, rt)
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), P.embedding(table.float(), ids.tolist()))
    head = build_part("head", {"kind": "linear", "vocab_size": vocab, "width": width, "weight": "h", "tied_to": "e"})
    assert head.tensors()[0].fallback == "e"
    head.bind({"h": table.cuda()}, rt)
    logits = head.forward(x.cuda(), rt)
    assert logits.dtype == torch.float32
    assert_close(logits, P.linear(x.float(), table.float()), dtype, "head")


# ---------------------------------------------------------------------------
# a toy architecture defined here: blocks whose mixer keeps a running sum per
# sequence, next to attention blocks; one layer runs twice, one reads another's cache
# ---------------------------------------------------------------------------

def _register_toy(mixer_kind="running_mean", architecture="ToyForCausalLM"):
    from nnis_amd.config import register_architecture
    from nnis_amd.models import ModelSpec, ScheduleEntry
    from nnis_amd.parts import Mixer, StateRequest, TensorSpec, register_part
    from nnis_amd.parts.linear import Projection

    class RunningMean(Mixer):
        """y_t = W * mean(x_0 .. x_t): the sum so far is the state."""

        def __init__(self, width, weight):
            self.width, self.weight_name, self.proj = width, weight, None

        def tensors(self):
            return [TensorSpec(self.weight_name, (self.width, self.width))]

        def bind(self, weights, rt):
            self.proj = Projection(weights[self.weight_name], rt)

        def cache_request(self):
            return StateRequest((self.width,), "float32")

        def forward(self, x, ctx, view, rt):
            means = torch.empty(x.shape, dtype=torch.float32, device=x.device)
            start = 0
            for slot, count, pos0 in zip(ctx.host_slots, ctx.host_new, ctx.host_pos0):
                sums = view.state[slot] + torch.cumsum(x[start:start + count].float(), dim=0)
                if not view.read_only:
                    view.state[slot] = sums[-1]
                steps = torch.arange(pos0 + 1, pos0 + count + 1, device=x.device, dtype=torch.float32)
                means[start:start + count] = sums / steps[:, None]
                start += count
            return self.proj(means.to(rt.dtype), rt)

    @dataclass(frozen=True)
    class ToyConfig:
        width: int
        vocab_size: int
        layers: int
        raw: dict

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["width"], raw["vocab_size"], raw["layers"], dict(raw))

    def toy_spec(cfg):
        w = cfg.width

        def block(index, mixer):
            p = f"blocks.{index}."
            return {"kind": "pre_norm", "width": w,
                    "norm1": {"kind": "rms", "width": w, "eps": 1e-5, "weight": p + "n1"}, "mixer": mixer,
                    "norm2": {"kind": "rms", "width": w, "eps": 1e-5, "weight": p + "n2"},
                    "feed_forward": {"kind": "gated", "width": w, "inner": 2 * w + 8, "gate": p + "g", "up": p + "u", "down": p + "d"}}

        layers = []
        for index in range(cfg.layers):
            p = f"blocks.{index}."
            if index % 2 == 0:
                mixer = {"kind": mixer_kind, "width": w, "weight": p + "mix"}
            else:
                mixer = {"kind": "causal_attention", "width": w, "heads": 2, "kv_heads": 1, "head_dim": 16,
                         "position": "rope", "q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"}
            layers.append(block(index, mixer))
        # layer 0 runs twice (its second run keeps state of its own); the last
        # entry runs layer 1 again on the cache that entry 1 filled
        schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(0), ScheduleEntry(1, reads_cache_of=1)]
        return ModelSpec(
            architecture=architecture, width=w, vocab_size=cfg.vocab_size, max_positions=256, stored_dtype="bfloat16",
            embedding={"kind": "table", "vocab_size": cfg.vocab_size, "width": w, "weight": "emb"},
            positions={"rope": {"kind": "rotary_half", "rot_dim": 16, "theta": 1000.0, "max_positions": 256}},
            layers=layers, schedule=schedule,
            final_norm={"kind": "rms", "width": w, "eps": 1e-5, "weight": "norm"},
            head={"kind": "linear", "vocab_size": cfg.vocab_size, "width": w, "weight": "head", "tied_to": None},
            config_json=cfg.raw)

    register_part("mixer", "running_mean", RunningMean, replace=True)
    register_architecture(architecture, ToyConfig, toy_spec, replace=True)


def _plain_toy(folder, ids):
    """The toy model on one whole sequence with the plain functions."""
    from safetensors import safe_open

    with safe_open(folder + "/model.safetensors", framework="pt") as handle:
        w = {n: handle.get_tensor(n).float() for n in handle.keys()}
    t, width = len(ids), w["emb"].shape[1]
    cos, sin = (torch.from_numpy(a) for a in P.rope_tables(256, 16, 1000.0))
    x = P.embedding(w["emb"], ids)

    def attention(p, h):
        q = P.rope_rotate_half(P.linear(h, w[p + "q"]).view(t, 2, 16), cos[:t], sin[:t])
        k = P.rope_rotate_half(P.linear(h, w[p + "k"]).view(t, 1, 16), cos[:t], sin[:t])
        v = P.linear(h, w[p + "v"]).view(t, 1, 16)
        return q, k, v

    kept = {}
    for entry, (layer, reads) in enumerate([(0, None), (1, None), (2, None), (0, None), (1, 1)]):
        p = f"blocks.{layer}."
        h = P.rms_norm(x, w[p + "n1"], 1e-5)
        if layer % 2 == 0:
            steps = torch.arange(1, t + 1, dtype=torch.float32)[:, None]
            mixed = P.linear(torch.cumsum(h, 0) / steps, w[p + "mix"])
        else:
            q, k, v = attention(p, h)
            if reads is None:
                kept[entry] = (k, v)
            else:
                k, v = kept[reads]
            mixed = P.linear(P.causal_attention(q, k, v, 0.25).reshape(t, 32), w[p + "o"])
        x = x + mixed
        x = x + P.swiglu(P.rms_norm(x, w[p + "n2"], 1e-5), w[p + "g"], w[p + "u"], w[p + "d"])
    return P.linear(P.rms_norm(x, w["norm"], 1e-5), w["head"])


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_architecture_with_a_stateful_mixer(tmp_path, dtype):
    import nnis_amd
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry

    _register_toy()
    folder = str(tmp_path / "toy")
    raw = {"architectures": ["ToyForCausalLM"], "model_type": "toy", "width": 48, "vocab_size": 211, "layers": 3}
    nnis_amd.write_random_model(folder, raw, seed=3)
    engine = load_engine(folder, dtype=dtype, max_tokens=512)
    # two attention entries keep keys and values (the third reads the second's); three keep a running sum
    assert len(engine.cache.kv_groups) == 1 and len(engine.cache.kv_groups[0].entries) == 1
    assert sorted(engine.cache.state_regions) == ["entry0", "entry2", "entry3"]
    rng = np.random.default_rng(0)
    a, b = rng.integers(0, 211, size=50).tolist(), rng.integers(0, 211, size=13).tolist()
    want_a, want_b = _plain_toy(folder, a), _plain_toy(folder, b)
    sa, sb = engine.start_sequence(), engine.start_sequence()
    rows = engine.step([StepEntry(sa, a[:40], list(range(40))), StepEntry(sb, b[:3], [0, 1, 2])]).cpu()
    assert_close(rows[:40], want_a[:40], dtype, "toy prompt a")
    assert_close(rows[40:], want_b[:3], dtype, "toy prompt b")
    for i in range(10):
        rows = engine.step([StepEntry(sb, [b[3 + i]], [0]), StepEntry(sa, [a[40 + i]], [0])]).cpu()
        assert_close(rows[0], want_b[3 + i], dtype, f"toy decode b {i}")
        assert_close(rows[1], want_a[40 + i], dtype, f"toy decode a {i}")
    # a slot used again starts from zero state
    engine.end_sequence(sa)
    again = engine.start_sequence()
    assert again == sa
    rows = engine.step([StepEntry(again, b, list(range(13)))]).cpu()
    assert_close(rows, want_b, dtype, "toy reused slot")


# ---------------------------------------------------------------------------
# the same architecture with the running mean as a kernel of the test's own
# (tests/toy_running_mean.hip, a kernel module that the test registers) that
# reads the step from device memory and a work list that the mixer makes on
# the host: steps of prompts and of single tokens are replayed from graphs,
# with no word about this mixer, its list or its module in the library
# ---------------------------------------------------------------------------

def _register_kernel_toy():
    import ctypes
    import os

    from nnis_amd.kernels import lib, ops
    from nnis_amd.parts import Mixer, StateRequest, TensorSpec, register_part
    from nnis_amd.parts.linear import Projection

    lib.register_module("toy_mean", ["toy_running_mean.hip"], headers=["common.h"], directory=os.path.dirname(os.path.abspath(__file__)),
                        replace=True)
    # (common.h is the library's: found on the include path, hashed from the test's folder if a copy lay there)
    void, integer = ctypes.c_void_p, ctypes.c_int
    signatures = {"toy_running_mean": [void, void, void, void, void, void, void, integer, integer, integer, void]}

    def rows_of_sequences(counts, first_positions, padded):
        """The sequence of each row of a step of prompts; rows that belong to none name a sequence beyond the last."""
        rows = padded[1] if padded is not None else sum(counts)
        out = np.full(rows, len(counts) if padded is None else padded[0], dtype=np.int32)
        at = 0
        for index, count in enumerate(counts):
            out[at:at + count] = index
            at += count
        return out

    class RunningMeanKernel(Mixer):
        graph_safe = True  # the kernel reads slots and positions from the step's device arrays
        asked = []  # the plans the engine asked for

        def __init__(self, width, weight):
            self.width, self.weight_name, self.proj = width, weight, None

        def tensors(self):
            return [TensorSpec(self.weight_name, (self.width, self.width))]

        def bind(self, weights, rt):
            self.proj = Projection(weights[self.weight_name], rt)
            self.lib = ops.bind("toy_mean", signatures)

        def cache_request(self):
            return StateRequest((self.width,), "float32")

        def prompt_plan(self, batch, rows, longest, rt):
            type(self).asked.append((batch, rows, longest))
            return ("toy", rows > 64)  # (it launches the same way always; the plan only shows that it is asked and kept)

        def forward(self, x, ctx, view, rt):
            assert not view.read_only
            x = x.float().contiguous()
            y = torch.empty_like(x)
            row_seq = None if ctx.decode else ctx.lists.device_list(("toy_rows",), rows_of_sequences)
            ops.check(self.lib, self.lib.toy_running_mean(
                x.data_ptr(), None if row_seq is None else row_seq.data_ptr(), ctx.seq_start.data_ptr(), ctx.seq_slot.data_ptr(),
                ctx.tok_pos.data_ptr(), view.state.data_ptr(), y.data_ptr(), ctx.tokens, ctx.batch, self.width, ops.stream()))
            return self.proj(y.to(rt.dtype), rt)

    register_part("mixer", "running_mean_kernel", RunningMeanKernel, replace=True)
    _register_toy("running_mean_kernel", "ToyKernelForCausalLM")
    return RunningMeanKernel


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_a_kernel_and_a_list_of_its_own_is_replayed_from_graphs(tmp_path, dtype):
    import nnis_amd
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry

    mixer_class = _register_kernel_toy()
    folder = str(tmp_path / "toy")
    raw = {"architectures": ["ToyKernelForCausalLM"], "model_type": "toy", "width": 48, "vocab_size": 211, "layers": 3}
    nnis_amd.write_random_model(folder, raw, seed=4)
    engine = load_engine(folder, dtype=dtype, max_tokens=2048)
    assert engine.use_graphs
    rng = np.random.default_rng(2)

    def run(lengths, decode):
        """Prompts of these lengths in one step (all their logits), then ``decode`` steps of one token each."""
        sequences = [rng.integers(0, 211, size=n + decode).tolist() for n in lengths]
        want = [_plain_toy(folder, ids) for ids in sequences]
        slots = [engine.start_sequence() for _ in sequences]
        rows = engine.step([StepEntry(s, ids[:n], list(range(n))) for s, ids, n in zip(slots, sequences, lengths)]).cpu()
        at = 0
        for w, n in zip(want, lengths):
            assert_close(rows[at:at + n], w[:n], dtype, f"prompts of {lengths}")
            at += n
        for step in range(decode):
            rows = engine.step([StepEntry(s, [ids[n + step]], [0]) for s, ids, n in zip(slots, sequences, lengths)]).cpu()
            for j, (w, n) in enumerate(zip(want, lengths)):
                assert_close(rows[j], w[n + step], dtype, f"decode step {step} after prompts of {lengths}")
        for slot in slots:
            engine.end_sequence(slot)

    run([37, 5, 70], 3)  # launched
    run([37, 5, 70], 0)  # from fixed buffers, captured
    graphs = engine._prefill_graphs.graphs
    (key,) = list(graphs)
    assert key[:3] == (3, 128, 112) and "'toy', True" in repr(key[3])  # the toy's plan is part of the shape
    graph = graphs[key]
    assert ("toy_rows",) in graph.list_keys  # the toy's list lies in the graph's buffers, beside the attention's own
    if dtype == "bfloat16":
        assert any(k[0] == "attention_tiles" for k in graph.list_keys)
    assert mixer_class.asked and mixer_class.asked[-1][:2] == (3, 128)
    run([37, 5, 70], 2)  # replayed, in other slots' state rows than before
    run([30, 42, 40], 2)  # the same shape, divided otherwise: the lists are made anew for it
    run([70, 1, 41], 0)
    assert list(graphs) == [key] and engine._graphs is not None and engine._graphs.graphs  # single tokens from graphs too


# ---------------------------------------------------------------------------
# a second toy architecture: a feed-forward that routes each token to one of
# several experts, positions learned and added to the embedding (no rotation),
# and a norm of another kind (centred) -- all three defined here
# ---------------------------------------------------------------------------

def _register_routed_toy():
    from nnis_amd.config import register_architecture
    from nnis_amd.models import ModelSpec, ScheduleEntry
    from nnis_amd.parts import FeedForward, Norm, PositionEncoding, TensorSpec, register_part
    from nnis_amd.parts.linear import Projection

    class RoutedFeedForward(FeedForward):
        """y = p_e * W2_e relu(W1_e x) for the expert e with the largest router logit, p its softmax weight."""

        def __init__(self, width, inner, experts, router, first, second):
            self.width, self.inner, self.experts = width, inner, experts
            self.names = (router, first, second)

        def tensors(self):
            router, first, second = self.names
            specs = [TensorSpec(router, (self.experts, self.width))]
            for e in range(self.experts):
                specs += [TensorSpec(f"{first}.{e}", (self.inner, self.width)), TensorSpec(f"{second}.{e}", (self.width, self.inner))]
            return specs

        def bind(self, weights, rt):
            router, first, second = self.names
            self.router = weights[router].float()  # router logits are taken in 32-bit
            self.first = [Projection(weights[f"{first}.{e}"], rt) for e in range(self.experts)]
            self.second = [Projection(weights[f"{second}.{e}"], rt) for e in range(self.experts)]

        def forward(self, x, ctx, rt):
            logits = x.float() @ self.router.t()
            weight, chosen = torch.softmax(logits, dim=-1).max(dim=-1)
            y = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
            for e in range(self.experts):
                rows = (chosen == e).nonzero().flatten()
                if rows.numel():
                    hidden = torch.relu(self.first[e](x[rows].contiguous(), rt))
                    y[rows] = self.second[e](hidden, rt).float() * weight[rows, None]
            return y.to(rt.dtype)

    class LearnedPositions(PositionEncoding):
        """x_t += table[position of t]."""

        def __init__(self, width, max_positions, weight):
            self.width, self.max_positions, self.weight_name = width, max_positions, weight

        def tensors(self):
            return [TensorSpec(self.weight_name, (self.max_positions, self.width))]

        def bind(self, weights, rt):
            self.table = weights[self.weight_name].float()

        def embed(self, x, ctx, rt):
            live = ctx.tok_slot[:x.shape[0]] >= 0
            rows = self.table[ctx.tok_pos[:x.shape[0]].long().clamp(min=0)]
            return x + rows * live[:, None]

    class CentredNorm(Norm):
        """(x - mean) / sqrt(var + eps) * weight."""

        def __init__(self, width, eps, weight):
            self.width, self.eps, self.weight_name = width, eps, weight

        def tensors(self):
            return [TensorSpec(self.weight_name, (self.width,), init="gain")]

        def bind(self, weights, rt):
            self.gain = weights[self.weight_name].float()

        def forward(self, x, rt, rows=None):
            x = x.float() if rows is None else x.float()[rows.long()]
            centred = x - x.mean(dim=-1, keepdim=True)
            return (centred * torch.rsqrt(centred.pow(2).mean(dim=-1, keepdim=True) + self.eps) * self.gain).to(rt.dtype)

        def add_forward(self, residual, delta, rt, rows=None):
            residual += delta.float()
            return self.forward(residual, rt, rows)

    @dataclass(frozen=True)
    class RoutedConfig:
        width: int
        vocab_size: int
        layers: int
        experts: int
        raw: dict

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["width"], raw["vocab_size"], raw["layers"], raw["experts"], dict(raw))

    def routed_spec(cfg):
        w = cfg.width
        layers = []
        for index in range(cfg.layers):
            p = f"h.{index}."
            layers.append({
                "kind": "pre_norm", "width": w,
                "norm1": {"kind": "centred", "width": w, "eps": 1e-4, "weight": p + "ln1"},
                "mixer": {"kind": "causal_attention", "width": w, "heads": 3, "kv_heads": 3, "head_dim": 16, "position": None,
                          "q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"},
                "norm2": {"kind": "centred", "width": w, "eps": 1e-4, "weight": p + "ln2"},
                # dense in the even layers, routed in the odd ones
                "feed_forward": ({"kind": "gated", "width": w, "inner": 72, "gate": p + "g", "up": p + "u", "down": p + "d"}
                                 if index % 2 == 0 else
                                 {"kind": "routed_relu", "width": w, "inner": 40, "experts": cfg.experts, "router": p + "router",
                                  "first": p + "w1", "second": p + "w2"})})
        return ModelSpec(
            architecture="RoutedToyForCausalLM", width=w, vocab_size=cfg.vocab_size, max_positions=128, stored_dtype="bfloat16",
            embedding={"kind": "table", "vocab_size": cfg.vocab_size, "width": w, "weight": "wte"},
            positions={"learned": {"kind": "learned", "width": w, "max_positions": 128, "weight": "wpe"}},
            layers=layers, schedule=[ScheduleEntry(i) for i in range(cfg.layers)],
            final_norm={"kind": "centred", "width": w, "eps": 1e-4, "weight": "ln_f"},
            head={"kind": "linear", "vocab_size": cfg.vocab_size, "width": w, "weight": "head", "tied_to": "wte"},
            config_json=cfg.raw)

    register_part("feed_forward", "routed_relu", RoutedFeedForward, replace=True)
    register_part("position", "learned", LearnedPositions, replace=True)
    register_part("norm", "centred", CentredNorm, replace=True)
    register_architecture("RoutedToyForCausalLM", RoutedConfig, routed_spec, replace=True)


def _plain_routed_toy(folder, ids, layers, experts):
    from safetensors import safe_open

    with safe_open(folder + "/model.safetensors", framework="pt") as handle:
        w = {n: handle.get_tensor(n).float() for n in handle.keys()}
    t = len(ids)

    def norm(x, gain):
        centred = x - x.mean(dim=-1, keepdim=True)
        return centred * torch.rsqrt(centred.pow(2).mean(dim=-1, keepdim=True) + 1e-4) * gain

    x = P.embedding(w["wte"], ids) + w["wpe"][:t]
    chosen_all = []
    for layer in range(layers):
        p = f"h.{layer}."
        h = norm(x, w[p + "ln1"])
        q, k, v = (P.linear(h, w[p + n]).view(t, 3, 16) for n in "qkv")
        x = x + P.linear(P.causal_attention(q, k, v, 0.25).reshape(t, 48), w[p + "o"])
        h = norm(x, w[p + "ln2"])
        if layer % 2 == 0:
            x = x + P.swiglu(h, w[p + "g"], w[p + "u"], w[p + "d"])
        else:
            weight, chosen = torch.softmax(P.linear(h, w[p + "router"]), dim=-1).max(dim=-1)
            chosen_all.append(chosen)
            y = torch.stack([P.linear(torch.relu(P.linear(h[i:i + 1], w[f"{p}w1.{int(e)}"])), w[f"{p}w2.{int(e)}"])[0]
                             for i, e in enumerate(chosen)])
            x = x + y * weight[:, None]
    return P.linear(norm(x, w["ln_f"]), w["wte"]), chosen_all


def test_toy_architecture_with_routing_and_learned_positions(tmp_path):
    """A feed-forward with routing in some layers and a dense one in others, positions added to the
    embedding, attention without rotation and a norm of another kind: registered, built, loaded and
    stepped (whole prompts of unequal lengths, then token by token) without a change to the library."""
    import nnis_amd
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry

    _register_routed_toy()
    folder = str(tmp_path / "routed")
    raw = {"architectures": ["RoutedToyForCausalLM"], "model_type": "routed_toy", "width": 48, "vocab_size": 157, "layers": 4,
           "experts": 3}
    nnis_amd.write_random_model(folder, raw, seed=11)
    # random routers of N(0, 0.02) would leave every choice a near tie: make them decisive
    from nnis_amd.weights.safetensors_io import SafetensorsFile, write_safetensors

    stored = SafetensorsFile(folder + "/model.safetensors")
    tensors = {name: stored.tensor(name).clone() for name in stored.names()}
    stored.close()
    for name in tensors:
        if name.endswith("router"):
            tensors[name] = (tensors[name].float() * 200).to(tensors[name].dtype)
    write_safetensors(folder + "/model.safetensors", tensors.items())
    engine = load_engine(folder, dtype="float32", max_tokens=512)
    rng = np.random.default_rng(5)
    a, b = rng.integers(0, 157, size=37).tolist(), rng.integers(0, 157, size=9).tolist()
    (want_a, chosen_a), (want_b, _) = _plain_routed_toy(folder, a, 4, 3), _plain_routed_toy(folder, b, 4, 3)
    assert all(len(set(c.tolist())) > 1 for c in chosen_a), "the test's tokens must reach more than one expert"
    sa, sb = engine.start_sequence(), engine.start_sequence()
    rows = engine.step([StepEntry(sa, a[:30], list(range(30))), StepEntry(sb, b[:2], [0, 1])]).cpu()
    assert_close(rows[:30], want_a[:30], "float32", "routed prompt a")
    assert_close(rows[30:], want_b[:2], "float32", "routed prompt b")
    for i in range(7):
        rows = engine.step([StepEntry(sb, [b[2 + i]], [0]), StepEntry(sa, [a[30 + i]], [0])]).cpu()
        assert_close(rows[0], want_b[2 + i], "float32", f"routed decode b {i}")
        assert_close(rows[1], want_a[30 + i], "float32", f"routed decode a {i}")


# ---------------------------------------------------------------------------
# a third toy architecture: layers that read all keys next to layers that read
# a window of them, with head sizes of their own -- two groups of the cache
# ---------------------------------------------------------------------------

_WINDOW = 40


def _register_windowed_toy():
    from nnis_amd.config import register_architecture
    from nnis_amd.models import ModelSpec, ScheduleEntry

    @dataclass(frozen=True)
    class WindowedConfig:
        width: int
        vocab_size: int
        layers: int
        raw: dict

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["width"], raw["vocab_size"], raw["layers"], dict(raw))

    def windowed_spec(cfg):
        w = cfg.width
        layers = []
        for index in range(cfg.layers):
            p = f"l.{index}."
            wide = index % 2 == 0  # even layers: all keys, 4 heads of 16 on 2; odd: a window, 2 heads of 32 on 1
            layers.append({
                "kind": "pre_norm", "width": w,
                "norm1": {"kind": "rms", "width": w, "eps": 1e-5, "weight": p + "n1"},
                "mixer": {"kind": "causal_attention", "width": w, "heads": 4 if wide else 2, "kv_heads": 2 if wide else 1,
                          "head_dim": 16 if wide else 32, "position": "rope16" if wide else "rope32",
                          "window": None if wide else _WINDOW, "q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"},
                "norm2": {"kind": "rms", "width": w, "eps": 1e-5, "weight": p + "n2"},
                "feed_forward": {"kind": "gated", "width": w, "inner": 88, "gate": p + "g", "up": p + "u", "down": p + "d"}})
        return ModelSpec(
            architecture="WindowedToyForCausalLM", width=w, vocab_size=cfg.vocab_size, max_positions=256, stored_dtype="bfloat16",
            embedding={"kind": "table", "vocab_size": cfg.vocab_size, "width": w, "weight": "emb"},
            positions={"rope16": {"kind": "rotary_half", "rot_dim": 16, "theta": 10000.0, "max_positions": 256},
                       "rope32": {"kind": "rotary_half", "rot_dim": 32, "theta": 500.0, "max_positions": 256}},
            layers=layers, schedule=[ScheduleEntry(i) for i in range(cfg.layers)],
            final_norm={"kind": "rms", "width": w, "eps": 1e-5, "weight": "norm"},
            head={"kind": "linear", "vocab_size": cfg.vocab_size, "width": w, "weight": "head", "tied_to": "emb"},
            config_json=cfg.raw)

    register_architecture("WindowedToyForCausalLM", WindowedConfig, windowed_spec, replace=True)


def _plain_windowed_toy(folder, ids, layers, window=_WINDOW):
    from safetensors import safe_open

    with safe_open(folder + "/model.safetensors", framework="pt") as handle:
        w = {n: handle.get_tensor(n).float() for n in handle.keys()}
    t = len(ids)
    x = P.embedding(w["emb"], ids)
    for layer in range(layers):
        p = f"l.{layer}."
        wide = layer % 2 == 0
        heads, kv_heads, hd, theta = (4, 2, 16, 10000.0) if wide else (2, 1, 32, 500.0)
        cos, sin = (torch.from_numpy(a)[:t] for a in P.rope_tables(256, hd, theta))
        h = P.rms_norm(x, w[p + "n1"], 1e-5)
        q = P.rope_rotate_half(P.linear(h, w[p + "q"]).view(t, heads, hd), cos, sin)
        k = P.rope_rotate_half(P.linear(h, w[p + "k"]).view(t, kv_heads, hd), cos, sin)
        v = P.linear(h, w[p + "v"]).view(t, kv_heads, hd)
        if wide:
            mixed = P.causal_attention(q, k, v, hd ** -0.5)
        else:  # the query at p reads keys p - window + 1 .. p
            k_all, v_all = (a.repeat_interleave(heads // kv_heads, dim=1) for a in (k, v))
            scores = torch.einsum("qhd,khd->hqk", q, k_all) * hd ** -0.5
            place = torch.arange(t)
            seen = (place[None, :] <= place[:, None]) & (place[None, :] > place[:, None] - window)
            scores = scores.masked_fill(~seen[None], float("-inf"))
            mixed = torch.einsum("hqk,khd->qhd", torch.softmax(scores, dim=-1), v_all)
        x = x + P.linear(mixed.reshape(t, heads * hd), w[p + "o"])
        x = x + P.swiglu(P.rms_norm(x, w[p + "n2"], 1e-5), w[p + "g"], w[p + "u"], w[p + "d"])
    return P.linear(P.rms_norm(x, w["norm"], 1e-5), w["emb"])


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_architecture_with_windowed_layers(tmp_path, dtype):
    """Layers that keep all keys and layers that read a window of 40, with head sizes of their own: the cache
    gives each kind storage of its own, and prompts longer than the window, cut before and behind the
    window's edge, then decoded one by one across a page's edge, give the plain model's logits."""
    import nnis_amd
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry

    _register_windowed_toy()
    folder = str(tmp_path / "windowed")
    raw = {"architectures": ["WindowedToyForCausalLM"], "model_type": "windowed_toy", "width": 64, "vocab_size": 301, "layers": 4}
    nnis_amd.write_random_model(folder, raw, seed=21)
    engine = load_engine(folder, dtype=dtype, max_tokens=512)
    groups = engine.cache.kv_groups
    assert len(groups) == 2 and sorted(g.request.window or 0 for g in groups) == [0, _WINDOW]
    assert sorted(len(g.entries) for g in groups) == [2, 2]
    rng = np.random.default_rng(9)
    a, b = rng.integers(0, 301, size=150).tolist(), rng.integers(0, 301, size=45).tolist()
    want_a, want_b = _plain_windowed_toy(folder, a, 4), _plain_windowed_toy(folder, b, 4)
    # the window matters: with one key more or less in it the plain logits move by far more than the 32-bit
    # bound (the window's edge in bfloat16 is the kernel tests' matter: a loud key just outside and just inside)
    for other in (_WINDOW - 1, _WINDOW + 1):
        moved = (_plain_windowed_toy(folder, a, 4, window=other)[_WINDOW:] - want_a[_WINDOW:]).abs().max(dim=-1).values
        assert moved.min().item() > 20 * tolerance("float32")[0], moved.min().item()
    sa, sb = engine.start_sequence(), engine.start_sequence()
    rows = engine.step([StepEntry(sa, a[:30], list(range(30))), StepEntry(sb, b[:41], list(range(41)))]).cpu()
    assert_close(rows[:30], want_a[:30], dtype, "windowed prompt a, inside the window")
    assert_close(rows[30:], want_b[:41], dtype, "windowed prompt b, one token beyond the window")
    rows = engine.step([StepEntry(sa, a[30:120], list(range(90)))]).cpu()  # a second run of tokens, across the window and a page
    assert_close(rows, want_a[30:120], dtype, "windowed continuation of a")
    for i in range(4):
        rows = engine.step([StepEntry(sb, [b[41 + i]], [0]), StepEntry(sa, [a[120 + i]], [0])]).cpu()
        assert_close(rows[0], want_b[41 + i], dtype, f"windowed decode b {i}")
        assert_close(rows[1], want_a[120 + i], dtype, f"windowed decode a {i}")
    engine.end_sequence(sb)
    for i in range(124, 150):  # alone, over the edge of the second page
        rows = engine.step([StepEntry(sa, [a[i]], [0])]).cpu()
        assert_close(rows[0], want_a[i], dtype, f"windowed decode a {i}")


# ---------------------------------------------------------------------------
# a fourth toy architecture: attention whose values are narrower than its keys
# (a cache need of its own shape), with a bias drawn by an init rule the test
# registers, a plan of its own for steps of single tokens, and a sequence that
# is cut back and goes on differently
# ---------------------------------------------------------------------------

def _register_narrow():
    from nnis_amd.cache.layout import k_offset, v_offset
    from nnis_amd.config import register_architecture
    from nnis_amd.models import ModelSpec, ScheduleEntry
    from nnis_amd.parts import Mixer, TensorSpec, register_part
    from nnis_amd.parts.base import KVRequest
    from nnis_amd.weights import register_init_rule

    register_init_rule("toy_tenth", lambda spec, generator, dtype: torch.full(tuple(spec.shape), 0.1, dtype=dtype), replace=True)
    KD, VD = 32, 16
    k_index = torch.tensor([[k_offset(t, c) for c in range(KD)] for t in range(64)])
    v_index = torch.tensor([[v_offset(c, t) for c in range(VD)] for t in range(64)])

    class NarrowValueAttention(Mixer):
        """One head, no rotation: y = W_o softmax(q k^T / sqrt(32)) v + bias, keys of 32 channels, values of 16."""

        planned = []  # what decode_plan was asked (the engine asks it only where steps are replayed from graphs)

        def __init__(self, width, q, k, v, o, bias):
            self.width, self.names, self.w = width, dict(q=q, k=k, v=v, o=o, bias=bias), None

        def tensors(self):
            n, w = self.names, self.width
            return [TensorSpec(n["q"], (KD, w)), TensorSpec(n["k"], (KD, w)), TensorSpec(n["v"], (VD, w)),
                    TensorSpec(n["o"], (w, VD)), TensorSpec(n["bias"], (w,), init="toy_tenth")]

        def bind(self, weights, rt):
            self.w = {key: weights[name].float() for key, name in self.names.items()}

        def cache_request(self):
            return KVRequest(1, KD, value_dim=VD)

        def decode_plan(self, batch, longest, rt):
            type(self).planned.append((batch, longest))
            return ("narrow", (longest + 63) // 64)

        def forward(self, x, ctx, view, rt):
            x = x.float()
            q, k, v = x @ self.w["q"].t(), x @ self.w["k"].t(), x @ self.w["v"].t()
            out = torch.empty(x.shape[0], VD, device=x.device)
            k_flat, v_flat = view.k_pages.view(view.k_pages.shape[0], -1), view.v_pages.view(view.v_pages.shape[0], -1)
            ki, vi = k_index.to(x.device), v_index.to(x.device)
            start = 0
            for slot, count, pos0 in zip(ctx.host_slots, ctx.host_new, ctx.host_pos0):
                table = view.block_table[slot].long()
                for i in range(count):  # the new tokens' keys and values into their pages
                    pos = pos0 + i
                    k_flat[table[pos // 64], ki[pos % 64]] = k[start + i].to(k_flat.dtype)
                    v_flat[table[pos // 64], vi[pos % 64]] = v[start + i].to(v_flat.dtype)
                total = pos0 + count
                pages = table[:(total + 63) // 64]
                keys = k_flat[pages][:, ki].reshape(-1, KD)[:total].float()
                values = v_flat[pages][:, vi].reshape(-1, VD)[:total].float()
                scores = (q[start:start + count] @ keys.t()) / math.sqrt(KD)
                mask = torch.arange(total, device=x.device)[None, :] > (pos0 + torch.arange(count, device=x.device))[:, None]
                out[start:start + count] = torch.softmax(scores.masked_fill(mask, float("-inf")), -1) @ values
                start += count
            return (out @ self.w["o"].t() + self.w["bias"]).to(rt.dtype)

    @dataclass(frozen=True)
    class NarrowConfig:
        raw: dict

        @classmethod
        def from_dict(cls, raw):
            return cls(dict(raw))

    def narrow_spec(cfg):
        w, vocab = cfg.raw["width"], cfg.raw["vocab_size"]
        layers = []
        for index in range(2):
            p = f"l{index}."
            layers.append({"kind": "pre_norm", "width": w,
                           "norm1": {"kind": "rms", "width": w, "eps": 1e-5, "weight": p + "n1"},
                           "mixer": {"kind": "narrow_value_attention", "width": w, "q": p + "q", "k": p + "k", "v": p + "v",
                                     "o": p + "o", "bias": p + "b"},
                           "norm2": {"kind": "rms", "width": w, "eps": 1e-5, "weight": p + "n2"},
                           "feed_forward": {"kind": "gated", "width": w, "inner": 3 * w, "gate": p + "g", "up": p + "u", "down": p + "d"}})
        return ModelSpec(
            architecture="NarrowForCausalLM", width=w, vocab_size=vocab, max_positions=256, stored_dtype="float32",
            embedding={"kind": "table", "vocab_size": vocab, "width": w, "weight": "emb"}, positions={},
            layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1)],
            final_norm={"kind": "rms", "width": w, "eps": 1e-5, "weight": "norm"},
            head={"kind": "linear", "vocab_size": vocab, "width": w, "weight": "head", "tied_to": None},
            config_json=cfg.raw)

    register_part("mixer", "narrow_value_attention", NarrowValueAttention, replace=True)
    register_architecture("NarrowForCausalLM", NarrowConfig, narrow_spec, replace=True)
    return NarrowValueAttention


def _plain_narrow(folder, ids):
    from safetensors import safe_open

    with safe_open(folder + "/model.safetensors", framework="pt") as handle:
        w = {n: handle.get_tensor(n).float() for n in handle.keys()}
    t = len(ids)
    x = P.embedding(w["emb"], ids)
    for index in range(2):
        p = f"l{index}."
        h = P.rms_norm(x, w[p + "n1"], 1e-5)
        q, k, v = P.linear(h, w[p + "q"]), P.linear(h, w[p + "k"]), P.linear(h, w[p + "v"])
        scores = (q @ k.t()) / math.sqrt(32)
        scores = scores.masked_fill(~torch.tril(torch.ones(t, t, dtype=torch.bool)), float("-inf"))
        x = x + P.linear(torch.softmax(scores, -1) @ v, w[p + "o"]) + w[p + "b"]
        x = x + P.swiglu(P.rms_norm(x, w[p + "n2"], 1e-5), w[p + "g"], w[p + "u"], w[p + "d"])
    return P.linear(P.rms_norm(x, w["norm"], 1e-5), w["head"])


def test_toy_architecture_with_narrow_values_and_a_sequence_cut_back(tmp_path):
    import nnis_amd
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.errors import InvalidInput
    from nnis_amd.weights import SafetensorsFile

    mixer_class = _register_narrow()
    folder = str(tmp_path / "narrow")
    raw = {"architectures": ["NarrowForCausalLM"], "model_type": "narrow", "width": 40, "vocab_size": 97}
    nnis_amd.write_random_model(folder, raw, seed=8)
    stored = SafetensorsFile(folder + "/model.safetensors")
    assert bool((stored.tensor("l1.b") == 0.1).all())  # drawn by the rule the test registered
    engine = load_engine(folder, dtype="float32", max_tokens=512)
    group, = engine.cache.kv_groups  # one need: keys of 32 channels, values of 16, storage of that shape
    assert group.k.shape[2:] == (1, 4, 64, 8) and group.v.shape[2:] == (1, 1, 2, 4, 16, 8)
    assert not engine.use_graphs  # the toy mixer reads the step's lengths on the host
    assert engine.model.decode_plan(3, 130, engine.rt) == (("narrow", 3), ("narrow", 3)) and mixer_class.planned[-1] == (3, 130)
    rng = np.random.default_rng(1)
    a, b = rng.integers(0, 97, size=150).tolist(), rng.integers(0, 97, size=20).tolist()
    want_a, want_b = _plain_narrow(folder, a), _plain_narrow(folder, b)
    sa, sb = engine.start_sequence(), engine.start_sequence()
    rows = engine.step([StepEntry(sa, a[:140], list(range(140))), StepEntry(sb, b[:5], [4])]).cpu()
    assert_close(rows[:140], want_a[:140], "float32", "narrow prompt a")
    assert_close(rows[140], want_b[4], "float32", "narrow prompt b")
    for i in range(10):
        rows = engine.step([StepEntry(sa, [a[140 + i]], [0]), StepEntry(sb, [b[5 + i]], [0])]).cpu()
        assert_close(rows[0], want_a[140 + i], "float32", f"narrow decode a {i}")
        assert_close(rows[1], want_b[5 + i], "float32", f"narrow decode b {i}")
    # cut a back to 70 tokens (its third page goes back to the cache) and go on with other tokens
    free = engine.free_pages()
    engine.truncate(sa, 70)
    assert engine.length(sa) == 70 and engine.free_pages() == free + 1
    with pytest.raises(InvalidInput):
        engine.truncate(sa, 71)
    other = a[:70] + rng.integers(0, 97, size=70).tolist()
    want_other = _plain_narrow(folder, other)
    rows = engine.step([StepEntry(sa, other[70:], list(range(70)))]).cpu()
    assert_close(rows, want_other[70:], "float32", "narrow sequence cut back and continued")
    engine.reset(sb)
    rows = engine.step([StepEntry(sb, a[:9], [8])]).cpu()
    assert_close(rows[0], want_a[8], "float32", "narrow slot reset and used again")
