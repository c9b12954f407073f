"""Decode and prefill throughput of the Llama engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

Default run: the SmolLM2-135M layer sizes (30 layers, hidden 576, 9 query and 3
key/value heads of 64, inner 1536, vocabulary 49152, tied head) with random
weights, a batch of 8 sequences whose prompts are uniform in [128, 2048]
tokens, in a cache sized for 8192 tokens per sequence.  A step is one decode
step of the whole batch through the generation path: token ids in, the model,
greedy selection on the device, token ids out to the host (which reads a
step's tokens while the next step, fed from the device, is under way, as the
generation loop does for greedy batches).  ``value`` is decoded tokens per
second over exactly K steps between two synchronisations; ``step_ms`` gives
the median, the least and the most of the steps' own times, taken with events
on the stream.  The prefill figure is one step over a 2,048-token prompt: the
time of a shape seen before (replayed from a captured graph where the engine
keeps one) and, beside it, of a shape seen for the first time.

``points`` holds, beside decode at batch 1 and 64 of the same shape, the same
four measurements at the SmolLM2-1.7B and TinyLlama-1.1B layer sizes (all
layers), each with the fraction of its roofline, and the TinyLlama workload
of 64 unequal prompts (16 to 1,024 tokens, prefilled in one step, decoded
until every sequence holds 2,048 tokens) run through ``nnis_amd.generate``.
For the SmolLM2 shapes there are further points at long contexts: decode at
batch 8 and 64 over prompts of 7,800 to 8,000 tokens (``*_ctx8k``) and a prompt
of 8,192 tokens in one step (``*_prefill_8192``).  A decode point is the
median of three windows of K steps, one after the other on the same batch; a
prefill figure is the median of seven runs of a shape seen before.
``--workload tinyllama-ragged`` runs that workload alone.

Peaks used for the fractions are the published MI355X ones: HBM 8 TB/s; dense
matrix rate 2.5 PFLOP/s for bfloat16, 157.3 TFLOP/s for 32-bit.
"""

import argparse
import json
import os
import subprocess
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FLOP_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}
NAMES = {"smollm2-135m": "SmolLM2-135M", "smollm2-1.7b": "SmolLM2-1.7B", "tinyllama-1.1b": "TinyLlama-1.1B", "llama-8b": "Llama-8B"}
POINT_SHAPES = ("smollm2-135m", "smollm2-1.7b", "tinyllama-1.1b")  # the shapes whose figures go into `points` beside the headline's


def step_flops(config, tokens_per_sequence, wanted_rows):
    """Multiply-adds x2 of one step over whole prompts from empty slots."""
    h, nq, nkv, hd = (config[k] for k in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim"))
    inner, vocab, layers = config["intermediate_size"], config["vocab_size"], config["num_hidden_layers"]
    per_token = 2 * ((nq + 2 * nkv) * hd * h + nq * hd * h + 3 * h * inner)
    total = 0
    for n in tokens_per_sequence:
        total += layers * (per_token * n + 2 * 2 * nq * hd * n * (n + 1) // 2)
    return total + 2 * wanted_rows * h * vocab


class Shape:
    """One model shape with random weights, loaded once; engines of any cache size share its weights."""

    def __init__(self, name, layers, dtype, seed, folder):
        import nnis_amd
        from nnis_amd.api import load_model
        from nnis_amd.config import preset

        self.name = name
        self.config = preset(name)
        self.layers_of_model = self.config["num_hidden_layers"]
        if layers:
            self.config["num_hidden_layers"] = layers
        self.dtype = dtype
        started = time.perf_counter()
        nnis_amd.write_random_model(folder, self.config, seed=seed)
        self.model, self.rt = load_model(folder, dtype=dtype)
        self.load_seconds = time.perf_counter() - started
        self.folder = folder
        self.context = self.config["max_position_embeddings"]
        self.vocab = self.config["vocab_size"]

    def engine(self, max_tokens, max_slots=None):
        from nnis_amd.engine.step import Engine

        return Engine(self.model, self.rt, max_tokens=max_tokens, max_slots=max_slots)


PROMPT_STEP_MOST_TOKENS = 16384  # a batch's prompts go in one step up to this many tokens, in several beyond


def decode_run(shape, rng, batch, steps, warmup, prompt_min, prompt_max, windows=1):
    """Prefills ``batch`` prompts (in one step where they are 16k tokens or fewer between them), then times
    ``windows`` windows of ``steps`` decode steps each, one after the other, and reports the median window.
    Returns a dict."""
    import torch

    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.sampling.device import DeviceSelector

    longest = min(prompt_max, shape.context - (windows + 1) * steps - warmup - 1)
    shortest = max(1, min(prompt_min, longest))
    lengths = rng.integers(shortest, longest + 1, size=batch).tolist()
    engine = shape.engine(batch * shape.context, max_slots=batch)  # every sequence may grow to the model's context
    selector = DeviceSelector(engine)
    slots = [engine.start_sequence() for _ in range(batch)]
    prompts = [rng.integers(0, shape.vocab, size=n).tolist() for n in lengths]
    rows, group, held = [], [], 0
    for slot, prompt in zip(slots, prompts):
        if group and held + len(prompt) > PROMPT_STEP_MOST_TOKENS:
            rows.append(engine.step([StepEntry(s, p, None) for s, p in group]))
            group, held = [], 0
        group.append((slot, prompt))
        held += len(prompt)
    rows.append(engine.step([StepEntry(s, p, None) for s, p in group]))
    logits = rows[0] if len(rows) == 1 else torch.cat(rows)
    greedy = [None] * batch
    sync = torch.cuda.synchronize
    if engine.use_graphs:
        # as the generation loop runs greedy batches: a step ahead of the host, which reads a
        # step's tokens while the next step, fed from the device, is under way
        pending = selector.select_start(logits, slots, greedy)

        def one_step(pending):
            following = selector.select_start(engine.step_from_device(slots, pending.device), slots, greedy)
            pending.result()
            return following

        def finish(pending):
            pending.result()
    else:
        pending = selector.select(logits, slots, greedy)

        def one_step(tokens):
            logits = engine.step_view([StepEntry(s, [t], None) for s, t in zip(slots, tokens)])
            return selector.select(logits, slots, greedy)

        def finish(tokens):
            pass

    for _ in range(warmup):
        pending = one_step(pending)
    finish(pending)
    # the graphs of the lengths that the timed steps (and the pass with events) reach are captured before the clock
    # starts: as the sequences grow a step may cross into another plan of the attention, whose first use costs 8 ms
    reached = max(engine.length(s) for s in slots)
    for ahead in range(1, min((windows + 1) * steps + 1, shape.context - reached) + 1):
        engine.prepare_decode(batch, reached + ahead)
    timed = []
    for _ in range(windows):
        sync()
        start = time.perf_counter()
        for _ in range(steps):
            pending = one_step(pending)
        finish(pending)
        sync()
        seconds = time.perf_counter() - start
        # (seconds, tokens held on average over the window's steps)
        timed.append((seconds, sum(engine.length(s) for s in slots) - batch * steps / 2.0))
    seconds, context_tokens = sorted(timed)[len(timed) // 2]
    # the steps' own times, in a pass of its own (an event on the stream after every step costs the step a little)
    spread = min(steps, shape.context - max(engine.length(s) for s in slots) - 1)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(spread + 1)]
    marks[0].record()
    for index in range(spread):
        pending = one_step(pending)
        marks[index + 1].record()
    finish(pending)
    sync()
    each = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(spread)) or [1000.0 * seconds / steps]
    step_bytes = engine.model.step_weight_bytes() + engine.cache.bytes_per_token() * context_tokens
    del engine, selector
    torch.cuda.empty_cache()
    per_step = seconds / steps
    return {
        "tokens_per_second": batch * steps / seconds, "ms_per_step": 1000.0 * per_step, "lengths": lengths,
        "prompt_min": shortest, "prompt_max": longest, "gbs": step_bytes / per_step / 1e9,
        "step_ms": {"median": round(each[len(each) // 2], 4), "min": round(each[0], 4), "max": round(each[-1], 4)},
    }


def prefill_run(shape, rng, tokens=2048):
    """One prompt of ``tokens`` tokens in one step, logits at the last place: the first time its shape comes
    and once it has come before."""
    import torch

    from nnis_amd.engine.batch import StepEntry

    tokens = min(tokens, shape.context)
    engine = shape.engine(tokens)
    prompt = rng.integers(0, shape.vocab, size=tokens).tolist()
    warm = rng.integers(0, shape.vocab, size=max(1, tokens // 2 - 7)).tolist()
    slot = engine.start_sequence()
    engine.step([StepEntry(slot, warm, None)])  # another shape: kernels loaded, buffers made
    engine.end_sequence(slot)
    times = []
    for _ in range(10):
        slot = engine.start_sequence()
        torch.cuda.synchronize()
        start = time.perf_counter()
        engine.step([StepEntry(slot, prompt, None)])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - start)
        engine.end_sequence(slot)
    del engine
    torch.cuda.empty_cache()
    seconds = sorted(times[3:])[3]  # the median of seven runs of a shape that has come before (and is captured, where it is)
    flops = step_flops(shape.config, [tokens], 1)
    return {"value": round(tokens / seconds, 1), "tokens": tokens, "ms": round(1000.0 * seconds, 3),
            "frac": round(flops / seconds / FLOP_PEAK[shape.dtype], 5), "first_ms": round(1000.0 * times[0], 3)}


def ragged_run(shape, rng, sequences=64, shortest=16, longest=1024):
    """BASELINE's fifth configuration through the generation loop: ``sequences`` prompts of unequal lengths in
    one step, each decoded greedily until it holds the model's context; the live set shrinks as they end."""
    import torch

    from nnis_amd.engine.generate import GenerationRequest, generate

    total = shape.context
    lengths = rng.integers(shortest, min(longest, total - 1) + 1, size=sequences).tolist()
    prompts = [rng.integers(0, shape.vocab, size=n).tolist() for n in lengths]
    engine = shape.engine(sequences * total, max_slots=sequences)
    generate(engine, [GenerationRequest(p[:16], 2, ()) for p in prompts[:4]])  # kernels loaded

    def timed(requests):
        torch.cuda.synchronize()
        start = time.perf_counter()
        results = generate(engine, requests, max_batch=sequences)
        torch.cuda.synchronize()
        return time.perf_counter() - start, results

    first, _ = timed([GenerationRequest(p, 1, ()) for p in prompts])  # the prompts' step and one selection
    whole, results = timed([GenerationRequest(p, total - len(p), ()) for p in prompts])
    generated = sum(len(r.tokens) for r in results)
    assert all(len(r.tokens) == total - n for r, n in zip(results, lengths))
    del engine
    torch.cuda.empty_cache()
    decode_seconds = max(whole - first, 1e-9)
    return {
        "sequences": sequences, "prompt_tokens": sum(lengths), "generated_tokens": generated,
        "prefill_tokens_per_second": round(sum(lengths) / first, 1), "prefill_ms": round(1000.0 * first, 2),
        "decode_tokens_per_second": round((generated - sequences) / decode_seconds, 1),
        "decode_steps": total - min(lengths) - 1, "seconds": round(whole, 3),
    }


def environment():
    import torch

    from nnis_amd.kernels import lib

    env = {"gpu": torch.cuda.get_device_name(0), "rocm": getattr(torch.version, "hip", None), "torch": torch.__version__,
           "kernels": lib.module_filename("core")}  # (named after a hash of the kernels' sources and flags)
    try:
        env["commit"] = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short=12", "HEAD"], capture_output=True, text=True,
                                       timeout=10).stdout.strip() or None
    except (OSError, subprocess.SubprocessError):
        env["commit"] = None
    if not env["commit"]:
        env["commit"] = os.environ.get("NNIS_COMMIT") or None  # a copy of the tree without its history: whoever made it may say
    return env


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--shape", default="smollm2-135m", choices=sorted(NAMES), help="layer sizes of the model")
    parser.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all of them)")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--no-points", action="store_true", help="only the headline: no further batches, shapes or workload")
    parser.add_argument("--no-other-shapes", action="store_true", help="points of the headline's shape only")
    parser.add_argument("--prompt-min", type=int, default=128, help="shortest prompt of the decode batches")
    parser.add_argument("--prompt-max", type=int, default=2048, help="longest prompt of the decode batches (within the context)")
    parser.add_argument("--workload", choices=["tinyllama-ragged"], help="run this workload alone")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import numpy as np

    rng = np.random.default_rng(args.seed)
    with tempfile.TemporaryDirectory() as folder:
        if args.workload == "tinyllama-ragged":
            shape = Shape("tinyllama-1.1b", args.layers, args.dtype, args.seed, folder)
            ragged = ragged_run(shape, rng)
            print(json.dumps({
                "metric": "TinyLlama-1.1B shape: 64 prompts of 16..1024 tokens in one step, decoded to 2048 tokens each",
                "value": ragged["decode_tokens_per_second"], "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
                "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
                "data": "synthetic: random weights N(0, 0.02) from a seed, uniform-random token ids",
                "config": {"model": "TinyLlama-1.1B shape (Llama)", "layers": shape.config["num_hidden_layers"],
                           "layers_of_model": shape.layers_of_model, "global_batch": 64, "seq_len": shape.context},
                "workload": ragged, "env": environment()}))
            return 0

        shape = Shape(args.shape, args.layers, args.dtype, args.seed, folder)
        head = decode_run(shape, rng, args.batch, args.steps, args.warmup, args.prompt_min, args.prompt_max)
        prefill = prefill_run(shape, rng)
        points = {}

        def point_run(shape, batch, prompt_min=args.prompt_min, prompt_max=args.prompt_max):
            """A point beside the headline: the median of three windows on one batch."""
            return decode_run(shape, rng, batch, args.steps, args.warmup, prompt_min, prompt_max, windows=3)

        def long_points(shape, prefix):
            """Contexts near the model's end: decode over prompts of 7,800 to 8,000 tokens, and a prompt of 8,192."""
            if shape.context < 8192:
                return
            for batch in (8, 64):
                run = point_run(shape, batch, 7800, 8000)
                points[f"{prefix}decode_b{batch}_ctx8k"] = round(run["tokens_per_second"], 1)
                points[f"{prefix}decode_b{batch}_ctx8k_hbm_frac"] = round(run["gbs"] / HBM_PEAK_GBS, 4)
            long_prefill = prefill_run(shape, rng, tokens=8192)
            points[f"{prefix}prefill_8192"] = long_prefill["value"]
            points[f"{prefix}prefill_8192_frac"] = long_prefill["frac"]

        if not args.no_points:
            for batch in (1, 64):
                run = point_run(shape, batch)
                points[f"decode_b{batch}"] = round(run["tokens_per_second"], 1)
                points[f"decode_b{batch}_hbm_frac"] = round(run["gbs"] / HBM_PEAK_GBS, 4)
            long_points(shape, "")
        config, layers, layers_of_model = shape.config, shape.config["num_hidden_layers"], shape.layers_of_model
        del shape
    if not args.no_points and not args.no_other_shapes:
        import torch

        for other in POINT_SHAPES:
            if other == args.shape:
                continue
            torch.cuda.empty_cache()
            with tempfile.TemporaryDirectory() as folder:
                shape = Shape(other, 0, args.dtype, args.seed, folder)
                for batch in (1, 8, 64):
                    run = point_run(shape, batch)
                    points[f"{other}_decode_b{batch}"] = round(run["tokens_per_second"], 1)
                    points[f"{other}_decode_b{batch}_hbm_frac"] = round(run["gbs"] / HBM_PEAK_GBS, 4)
                other_prefill = prefill_run(shape, rng)
                points[f"{other}_prefill_{other_prefill['tokens']}"] = other_prefill["value"]
                points[f"{other}_prefill_{other_prefill['tokens']}_frac"] = other_prefill["frac"]
                long_points(shape, f"{other}_")
                if other == "tinyllama-1.1b":
                    ragged = ragged_run(shape, rng)
                    points["tinyllama-1.1b_ragged64_prefill"] = ragged["prefill_tokens_per_second"]
                    points["tinyllama-1.1b_ragged64_decode"] = ragged["decode_tokens_per_second"]
                del shape

    record = {
        "metric": f"decode tok/s at batch {args.batch} ({NAMES[args.shape]} shape); prefill tok/s at {prefill['tokens']} tokens; "
                  "decode at batch 1 and 64, and the other shapes, in points",
        "value": round(head["tokens_per_second"], 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights N(0, 0.02) from a seed, uniform-random token ids",
        "config": {
            "model": f"{NAMES[args.shape]} shape (Llama)", "layers": layers, "layers_of_model": layers_of_model,
            "hidden": config["hidden_size"], "heads": config["num_attention_heads"], "kv_heads": config["num_key_value_heads"],
            "head_dim": config["head_dim"], "inner": config["intermediate_size"], "vocab": config["vocab_size"],
            "tied_head": config["tie_word_embeddings"], "context": config["max_position_embeddings"],
            "global_batch": args.batch, "seq_len": config["max_position_embeddings"], "prompt_min": head["prompt_min"],
            "prompt_max": head["prompt_max"], "mean_prompt": round(float(np.mean(head["lengths"])), 1),
            "parallelism": "single GPU", "sampling": "greedy on device",
        },
        "step_ms": head["step_ms"],
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(head["gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(head["gbs"] / HBM_PEAK_GBS, 5)},
        "points": points,
        "env": environment(),
    }
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
