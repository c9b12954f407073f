"""The command line's rules, without touching a GPU
(/root/reference/crates/nnis-cli/src/main.rs:1545-1720)."""

import pytest

from nnis_amd.cli import UsageError, main, parse_args


def test_generate_defaults():
    args = parse_args(["generate", "--model", "m", "--prompt", "hi"])
    assert (args.model_dir, args.prompts, args.device_ordinal, args.max_new_tokens) == ("m", ["hi"], 0, 16)
    assert not args.sample and not args.stream and args.seeds == [] and args.dtype == "bfloat16"
    args = parse_args(["generate", "--model", "m", "--prompt-ids", "5, 17,3", "--max-new-tokens", "4", "--device", "0",
                       "--sample", "--seed", "18446744073709551615", "--temperature", "0.8", "--top-k", "5",
                       "--top-p", "0.9", "--stream", "--dtype", "float32"])
    assert args.prompt_ids == [[5, 17, 3]] and args.seeds == [2**64 - 1] and args.temperature == 0.8
    assert args.top_k == 5 and args.top_p == 0.9 and args.stream and args.dtype == "float32"
    assert parse_args(["--help"]) == "help" and parse_args(["generate", "-h"]) == "help"


@pytest.mark.parametrize("argv, message", [
    (["generate", "--prompt", "x"], "missing --model"),
    (["generate", "--model", "m"], "missing --prompt"),
    (["generate", "--model", "m", "--prompt", "x", "--seed", "1"], "--seed requires --sample"),
    (["generate", "--model", "m", "--prompt", "x", "--temperature", "1"], "--temperature requires --sample"),
    (["generate", "--model", "m", "--prompt", "x", "--top-k", "1"], "--top-k requires --sample"),
    (["generate", "--model", "m", "--prompt", "x", "--top-p", "0.5"], "--top-p requires --sample"),
    (["generate", "--model", "m", "--prompt", "x", "--stream"], "--stream requires --sample"),
    (["generate", "--model", "m", "--prompt", "x", "--sample"], "--sample requires --seed"),
    (["generate", "--model", "m", "--prompt", "x", "--max-new-tokens", "0"], "greater than zero"),
    (["generate", "--model", "m", "--prompt", "x", "--max-new-tokens", "-3"], "invalid --max-new-tokens"),
    (["generate", "--model", "m", "--prompt", "x", "--device", "-1"], "non-negative"),
    (["generate", "--model", "m", "--prompt", "x", "--sample", "--seed", "-1"], "invalid --seed"),
    (["generate", "--model", "m", "--prompt", "x", "--sample", "--seed", "1", "--temperature", "0"], "finite and positive"),
    (["generate", "--model", "m", "--prompt", "x", "--sample", "--seed", "1", "--top-k", "0"], "greater than zero"),
    (["generate", "--model", "m", "--prompt", "x", "--sample", "--seed", "1", "--top-p", "1.5"], r"\(0, 1\]"),
    (["generate", "--model", "m", "--prompt", "x", "--bogus"], "unknown generate argument"),
    (["generate", "--model"], "--model requires"),
    (["generate", "--model", "m", "--prompt", "x", "--json"], "unknown generate argument"),
    (["generate", "--model", "m", "--prompt-ids", "a,b"], "invalid --prompt-ids"),
    (["generate-batch", "--model", "m", "--seed", "1"], "at least one --prompt"),
    (["generate-batch", "--model", "m", "--prompt", "a", "--prompt", "b", "--seed", "1"], "one --seed per --prompt"),
    (["generate-batch", "--model", "m", "--prompt", "a", "--seed", "1", "--sample"], "unknown generate-batch argument"),
    (["frobnicate"], "unknown command"),
])
def test_usage_errors(argv, message):
    with pytest.raises(UsageError, match=message):
        parse_args(argv)


def test_generate_batch_and_exit_codes(capsys):
    args = parse_args(["generate-batch", "--model", "m", "--prompt", "a", "--prompt-ids", "1,2", "--seed", "3",
                       "--seed", "4", "--json", "--temperature", "0.5"])
    assert args.batch and args.sample and args.seeds == [3, 4] and args.json and args.prompts == ["a", ""]
    assert args.prompt_ids == [[], [1, 2]]
    assert main(["generate", "--model", "m", "--prompt", "x", "--seed", "1"]) == 2  # usage error
    assert "requires --sample" in capsys.readouterr().err
    assert main(["--help"]) == 0
    assert "nnis generate --model DIR" in capsys.readouterr().out
