"""The measurement program's contract: what it prints for one GPU, what it does
when asked for more, and its count of a step's floating-point operations."""

import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def _run(*flags, timeout=600):
    return subprocess.run([sys.executable, BENCH, *flags], capture_output=True, text=True, timeout=timeout, cwd=ROOT)


def test_more_than_one_gpu_is_refused_in_one_line():
    done = _run("--gpus", "2", "--steps", "1", "--warmup", "0", timeout=120)
    assert done.returncode == 2
    assert len(done.stdout.strip().splitlines()) == 1 and "one GPU" in done.stdout


def test_step_flops_of_a_small_configuration():
    """Counted by hand for one layer: projections 2 * (q, k, v, o, gate, up, down) per token, scores and
    weighted values over the keys up to each token's own, the head on the wanted rows."""
    sys.path.insert(0, ROOT)
    import bench

    config = {"hidden_size": 8, "num_attention_heads": 2, "num_key_value_heads": 1, "head_dim": 4, "intermediate_size": 16,
              "vocab_size": 10, "num_hidden_layers": 1}
    per_token = 2 * ((2 + 2 * 1) * 4 * 8 + 2 * 4 * 8 + 3 * 8 * 16)
    attention = 2 * 2 * 2 * 4 * (3 * 4 // 2)  # scores and values, 2 heads of 4 channels, 1 + 2 + 3 keys
    assert bench.step_flops(config, [3], 1) == 3 * per_token + attention + 2 * 1 * 8 * 10
    two = dict(config, num_hidden_layers=2)
    assert bench.step_flops(two, [3, 1], 2) == 2 * (4 * per_token + attention + 2 * 2 * 2 * 4 * 1) + 2 * 2 * 8 * 10


@pytest.mark.gpu
def test_the_line_it_prints():
    """A short run at the headline's sizes with two of its layers: one JSON line with the fields the
    contract names, a flat ``config`` of at most 20 keys that names both layer counts, and figures that agree
    with each other."""
    done = _run("--layers", "2", "--steps", "6", "--warmup", "2", "--no-other-shapes")
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [line for line in done.stdout.splitlines() if line.strip()]
    assert len(lines) == 1
    record = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in record, key
    assert record["n_gpus"] == 1 and record["steps"] == 6 and record["warmup"] == 2 and record["higher_is_better"] is True
    assert record["dtype"] == "bf16" and record["unit"] == "tokens/s"
    config = record["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert config["layers"] == 2 and config["layers_of_model"] == 30 and config["global_batch"] == 8
    assert (config["hidden"], config["heads"], config["kv_heads"], config["head_dim"], config["inner"], config["vocab"]) == (576, 9, 3, 64, 1536, 49152)
    # tokens a second are the batch over a step's time (the times are printed rounded: to 4 and to 3 places)
    assert record["value"] == pytest.approx(8 / (record["ms_per_step"] / 1000.0), rel=1e-3 + 6e-5 / record["ms_per_step"])
    prefill = record["prefill"]
    assert prefill["tokens"] == 2048
    assert prefill["value"] == pytest.approx(2048 / (prefill["ms"] / 1000.0), rel=1e-3 + 6e-4 / prefill["ms"])
    assert 0 < prefill["frac"] < 1
    roofline = record["roofline"]
    assert roofline["bound"] == "hbm" and roofline["peak"] == 8000.0 and roofline["unit"] == "GB/s"
    assert roofline["frac"] == pytest.approx(roofline["achieved"] / roofline["peak"], rel=1e-3) and 0 < roofline["frac"] < 1
    assert record["points"]["decode_b1"] > 0 and record["points"]["decode_b64"] > record["points"]["decode_b1"]
