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
second.  The prefill figure is one step over a 2,048-token prompt.  Peaks used
for the fractions are the published MI355X ones: HBM 8 TB/s; dense matrix
rate 2.5 PFLOP/s for bfloat16, 157.3 TFLOP/s for 32-bit.
"""

import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FLOP_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}

SHAPES = {
    "smollm2-135m": dict(name="SmolLM2-135M", layers=30, hidden=576, heads=9, kv_heads=3, head_dim=64, inner=1536, vocab=49152,
                         rope_theta=100000.0, rms_norm_eps=1e-5, context=8192, tied=True),
    "smollm2-1.7b": dict(name="SmolLM2-1.7B", layers=24, hidden=2048, heads=32, kv_heads=32, head_dim=64, inner=8192, vocab=49152,
                         rope_theta=130000.0, rms_norm_eps=1e-5, context=8192, tied=True),
    "tinyllama-1.1b": dict(name="TinyLlama-1.1B", layers=22, hidden=2048, heads=32, kv_heads=4, head_dim=64, inner=5632,
                           vocab=32000, rope_theta=10000.0, rms_norm_eps=1e-5, context=2048, tied=False),
}
SHAPE = dict(SHAPES["smollm2-135m"])  # the default run's; --shape puts another in its place


def model_config(layers):
    return {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
        "num_hidden_layers": layers, "hidden_size": SHAPE["hidden"], "num_attention_heads": SHAPE["heads"],
        "num_key_value_heads": SHAPE["kv_heads"], "head_dim": SHAPE["head_dim"], "intermediate_size": SHAPE["inner"],
        "vocab_size": SHAPE["vocab"], "rope_theta": SHAPE["rope_theta"], "rms_norm_eps": SHAPE["rms_norm_eps"],
        "tie_word_embeddings": SHAPE["tied"], "max_position_embeddings": SHAPE["context"], "torch_dtype": "bfloat16",
        "eos_token_id": 0,
    }


def step_flops(layers, tokens_per_sequence, wanted_rows):
    """Multiply-adds x2 of one step over whole prompts from empty slots."""
    h, nq, nkv, hd, inner, vocab = (SHAPE[k] for k in ("hidden", "heads", "kv_heads", "head_dim", "inner", "vocab"))
    per_token = 2 * ((nq + 2 * nkv) * hd * h + nq * hd * h + 3 * h * inner)
    total = 0
    for n in tokens_per_sequence:
        total += layers * (per_token * n + 2 * 2 * nq * hd * n * (n + 1) // 2)
    return total + 2 * wanted_rows * h * vocab


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--shape", default="smollm2-135m", choices=sorted(SHAPES), help="layer sizes of the model")
    parser.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all of them)")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 decode points")
    parser.add_argument("--prompt-min", type=int, default=128, help="shortest prompt of the decode batches")
    parser.add_argument("--prompt-max", type=int, default=2048, help="longest prompt of the decode batches (within the context)")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    SHAPE.clear()
    SHAPE.update(SHAPES[args.shape])
    args.layers = args.layers or SHAPE["layers"]
    longest_prompt = min(args.prompt_max, SHAPE["context"] - args.steps - args.warmup - 1)
    shortest_prompt = max(1, min(args.prompt_min, longest_prompt))

    import numpy as np
    import torch

    import nnis_amd
    from nnis_amd.api import load_engine
    from nnis_amd.engine.batch import StepEntry
    from nnis_amd.sampling.device import DeviceSelector

    rng = np.random.default_rng(args.seed)
    with tempfile.TemporaryDirectory() as folder:
        nnis_amd.write_random_model(folder, model_config(args.layers), seed=args.seed)
        sync = torch.cuda.synchronize

        def decode_run(batch, steps, warmup):
            """Prefills ``batch`` prompts in one step, then times ``steps`` decode steps."""
            lengths = rng.integers(shortest_prompt, longest_prompt + 1, size=batch).tolist()
            room = batch * SHAPE["context"]  # every sequence may grow to the model's context
            engine = load_engine(folder, dtype=args.dtype, max_tokens=room)
            selector = DeviceSelector(engine)
            slots = [engine.start_sequence() for _ in range(batch)]
            prompts = [rng.integers(0, SHAPE["vocab"], size=n).tolist() for n in lengths]
            logits = engine.step([StepEntry(s, p, None) for s, p in zip(slots, prompts)])
            greedy = [None] * batch
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
            sync()
            start = time.perf_counter()
            for _ in range(steps):
                pending = one_step(pending)
            finish(pending)
            sync()
            seconds = time.perf_counter() - start
            context_tokens = sum(engine.length(s) for s in slots) - batch * steps / 2.0  # mean over the timed steps
            step_bytes = engine.model.step_weight_bytes() + engine.cache.bytes_per_token() * context_tokens
            del engine
            torch.cuda.empty_cache()
            return seconds, step_bytes, lengths

        seconds, step_bytes, lengths = decode_run(args.batch, args.steps, args.warmup)
        ms_per_step = 1000.0 * seconds / args.steps
        value = args.batch * args.steps / seconds
        achieved = step_bytes / (seconds / args.steps) / 1e9

        # prefill: 2,048 tokens of one sequence in one step, logits at the last place
        prefill_tokens = min(2048, SHAPE["context"])
        engine = load_engine(folder, dtype=args.dtype, max_tokens=prefill_tokens)
        prompt = rng.integers(0, SHAPE["vocab"], size=prefill_tokens).tolist()
        times = []
        for _ in range(4):
            slot = engine.start_sequence()
            sync()
            start = time.perf_counter()
            engine.step([StepEntry(slot, prompt, None)])
            sync()
            times.append(time.perf_counter() - start)
            engine.end_sequence(slot)
        prefill_seconds = min(times[1:])
        del engine
        torch.cuda.empty_cache()
        flops = step_flops(args.layers, [prefill_tokens], 1)

        points = {}
        if not args.no_points:
            for batch in (1, 64):
                s, _, _ = decode_run(batch, max(8, args.steps // 2), max(2, args.warmup // 2))
                points[f"decode_b{batch}"] = round(batch * max(8, args.steps // 2) / s, 1)

    record = {
        "metric": f"decode tok/s at batch {args.batch} ({SHAPE['name']} shape); prefill tok/s at {prefill_tokens} tokens; "
                  "decode at batch 1 and 64 in points",
        "value": round(value, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights N(0, 0.02) from a seed, uniform-random token ids",
        "config": {
            "model": f"{SHAPE['name']} shape (Llama)", "layers": args.layers, "layers_of_model": SHAPE["layers"],
            "hidden": SHAPE["hidden"], "heads": SHAPE["heads"], "kv_heads": SHAPE["kv_heads"], "head_dim": SHAPE["head_dim"],
            "inner": SHAPE["inner"], "vocab": SHAPE["vocab"], "tied_head": SHAPE["tied"], "context": SHAPE["context"],
            "global_batch": args.batch, "seq_len": SHAPE["context"], "prompt_min": shortest_prompt, "prompt_max": longest_prompt,
            "mean_prompt": round(float(np.mean(lengths)), 1), "parallelism": "single GPU", "sampling": "greedy on device",
        },
        "prefill": {
            "value": round(prefill_tokens / prefill_seconds, 1), "tokens": prefill_tokens,
            "ms": round(1000.0 * prefill_seconds, 3), "frac": round(flops / prefill_seconds / FLOP_PEAK[args.dtype], 5),
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 5)},
        "points": points,
    }
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
