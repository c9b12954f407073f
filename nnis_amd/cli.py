"""The ``nnis`` command line: ``generate`` and ``generate-batch`` with the
reference's option names, meanings, defaults and rules
(/root/reference/crates/nnis-cli/src/main.rs:179-498 parsing, :1140-1346
running, :1348-1391 exit codes: 0 success, 1 runtime failure, 2 usage error).

Additions of this library, because a model folder made from random weights has
no tokenizer: ``--prompt-ids 5,17,3`` gives a prompt as token ids (the output
is then ids too), ``--dtype`` picks the precision, ``--narrow-to-bfloat16``
rounds a checkpoint stored in 32-bit to bfloat16 as it is loaded (the
reference refuses to narrow implicitly,
/root/reference/crates/nnis-model/src/safetensors_loader.rs:610-624: here it
is the caller's explicit choice) and ``--max-tokens`` sizes the cache.  ``--tokenizer`` defaults to MODEL/tokenizer.json, as in the
reference's Hugging Face front end
(/root/reference/docs/HF_GENERATION_PROCESS.md:31).
"""

from __future__ import annotations

import json
import math
import os
import sys
from dataclasses import dataclass, field
from typing import List, Optional

DEFAULT_DEVICE_ORDINAL = 0
DEFAULT_MAX_NEW_TOKENS = 16
SAMPLING_POLICY_VERSION = 1
GENERATE_BATCH_JSON_SCHEMA_VERSION = 1

USAGE = """Usage:
  nnis generate --model DIR [--tokenizer FILE] (--prompt TEXT | --prompt-ids IDS) [--device N] [--max-new-tokens N] [--sample --seed U64] [--temperature F] [--top-k N] [--top-p F] [--stream] [--dtype bfloat16|float32] [--narrow-to-bfloat16] [--max-tokens N]
  nnis generate-batch --model DIR [--tokenizer FILE] (--prompt TEXT | --prompt-ids IDS) [--prompt ...] --seed U64 [--seed U64 ...] [--device N] [--max-new-tokens N] [--temperature F] [--top-k N] [--top-p F] [--json] [--dtype bfloat16|float32] [--narrow-to-bfloat16] [--max-tokens N]

Default decoding on `generate` is greedy. Opt-in `--sample` requires `--seed`. Optional `--temperature`, `--top-k`, and `--top-p` apply only with `--sample`. `--stream` is valid only with `--sample` and prints each token as it is emitted. The device ordinal defaults to 0.

`generate-batch` is always sampled and requires one `--seed` per prompt (no silent seed reuse). Shared optional `--temperature` / `--top-k` / `--top-p` apply to every request. The prompts are prefilled together in one step and decoded as one batch; a request that ends earlier leaves the batch. Human text by default; `--json` emits versioned JSON.

`--prompt-ids` takes comma-separated token ids instead of text; the output is then token ids. `--narrow-to-bfloat16` rounds weights stored in 32-bit to bfloat16 at load (with `--dtype bfloat16`)."""


class UsageError(Exception):
    pass


@dataclass
class GenerateArgs:
    model_dir: str
    tokenizer_file: Optional[str]
    prompts: List[str]
    prompt_ids: List[List[int]]
    device_ordinal: int = DEFAULT_DEVICE_ORDINAL
    max_new_tokens: int = DEFAULT_MAX_NEW_TOKENS
    sample: bool = False
    stream: bool = False
    seeds: List[int] = field(default_factory=list)
    temperature: Optional[float] = None
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    json: bool = False
    dtype: str = "bfloat16"
    narrow_to_bfloat16: bool = False
    max_tokens: Optional[int] = None
    batch: bool = False


def _int(flag: str, raw: str, minimum: Optional[int] = None) -> int:
    try:
        value = int(raw, 10)
    except ValueError:
        raise UsageError(f"invalid {flag} {raw!r}: not an integer") from None
    if minimum is not None and value < minimum:
        raise UsageError(f"invalid {flag} {raw!r}: must be at least {minimum}")
    return value


def _positive_float(flag: str, raw: str) -> float:
    try:
        value = float(raw)
    except ValueError:
        raise UsageError(f"invalid {flag} {raw!r}: not a number") from None
    if not math.isfinite(value) or value <= 0.0:
        raise UsageError(f"{flag} must be finite and positive; got {raw}")
    return value


def _ids(raw: str) -> List[int]:
    try:
        ids = [int(part, 10) for part in raw.replace(" ", "").split(",") if part != ""]
    except ValueError:
        raise UsageError(f"invalid --prompt-ids {raw!r}: expected comma-separated integers") from None
    if not ids:
        raise UsageError("--prompt-ids requires at least one token id")
    return ids


def parse_args(argv: List[str]):
    """Returns ``"help"`` or a ``GenerateArgs``; raises ``UsageError``."""
    if not argv or argv[0] in ("--help", "-h"):
        return "help"
    command, rest = argv[0], list(argv[1:])
    if command not in ("generate", "generate-batch"):
        raise UsageError(f"unknown command {command!r}\n\n{USAGE}")
    batch = command == "generate-batch"
    args = GenerateArgs(model_dir="", tokenizer_file=None, prompts=[], prompt_ids=[], batch=batch)
    model_dir = None
    it = iter(rest)

    def value(flag: str, what: str) -> str:
        try:
            return next(it)
        except StopIteration:
            raise UsageError(f"{flag} requires {what}") from None

    for argument in it:
        if argument == "--model":
            model_dir = value("--model", "a directory")
        elif argument == "--tokenizer":
            args.tokenizer_file = value("--tokenizer", "a file")
        elif argument == "--prompt":
            text = value("--prompt", "text")
            if not batch and (args.prompts or args.prompt_ids):
                raise UsageError("generate takes one prompt; use generate-batch for several")
            args.prompts.append(text)
            args.prompt_ids.append([])
        elif argument == "--prompt-ids":
            ids = _ids(value("--prompt-ids", "comma-separated token ids"))
            if not batch and (args.prompts or args.prompt_ids):
                raise UsageError("generate takes one prompt; use generate-batch for several")
            args.prompts.append("")
            args.prompt_ids.append(ids)
        elif argument == "--device":
            raw = value("--device", "an integer ordinal")
            args.device_ordinal = _int("--device", raw)
            if args.device_ordinal < 0:
                raise UsageError("--device must be a non-negative device ordinal")
        elif argument == "--max-new-tokens":
            raw = value("--max-new-tokens", "an integer")
            args.max_new_tokens = _int("--max-new-tokens", raw, 0)
            if args.max_new_tokens == 0:
                raise UsageError("--max-new-tokens must be greater than zero")
        elif argument == "--sample" and not batch:
            args.sample = True
        elif argument == "--stream" and not batch:
            args.stream = True
        elif argument == "--json" and batch:
            args.json = True
        elif argument == "--seed":
            raw = value("--seed", "an unsigned integer")
            seed = _int("--seed", raw, 0)
            if seed >= (1 << 64):
                raise UsageError(f"invalid --seed {raw!r}: does not fit 64 bits")
            if not batch and args.seeds:
                args.seeds[0] = seed
            else:
                args.seeds.append(seed)
        elif argument == "--temperature":
            args.temperature = _positive_float("--temperature", value("--temperature", "a float"))
        elif argument == "--top-k":
            raw = value("--top-k", "an integer")
            args.top_k = _int("--top-k", raw, 0)
            if args.top_k == 0:
                raise UsageError("--top-k must be greater than zero")
        elif argument == "--top-p":
            raw = value("--top-p", "a float")
            args.top_p = _positive_float("--top-p", raw)
            if args.top_p > 1.0:
                raise UsageError(f"--top-p must be in (0, 1]; got {raw}")
        elif argument == "--dtype":
            args.dtype = value("--dtype", "bfloat16 or float32")
            if args.dtype not in ("bfloat16", "float32"):
                raise UsageError(f"--dtype must be bfloat16 or float32; got {args.dtype}")
        elif argument == "--narrow-to-bfloat16":
            args.narrow_to_bfloat16 = True
        elif argument == "--max-tokens":
            args.max_tokens = _int("--max-tokens", value("--max-tokens", "an integer"), 1)
        elif argument in ("--help", "-h"):
            return "help"
        else:
            raise UsageError(f"unknown {command} argument {argument!r}\n\n{USAGE}")

    if batch:
        args.sample = True
        if not args.prompts:
            raise UsageError("generate-batch requires at least one --prompt TEXT")
        if len(args.seeds) != len(args.prompts):
            raise UsageError(
                f"generate-batch requires one --seed per --prompt (got {len(args.prompts)} prompts and "
                f"{len(args.seeds)} seeds); refusing silent seed reuse"
            )
    else:
        if args.stream and not args.sample:
            raise UsageError("--stream requires --sample")
        if args.sample and not args.seeds:
            raise UsageError("--sample requires --seed U64")
        if not args.sample:
            for present, flag in ((args.seeds, "--seed"), (args.temperature is not None, "--temperature"),
                                  (args.top_k is not None, "--top-k"), (args.top_p is not None, "--top-p")):
                if present:
                    raise UsageError(f"{flag} requires --sample")
    if model_dir is None:
        raise UsageError("missing --model DIR")
    args.model_dir = model_dir
    if not args.prompts:
        raise UsageError("missing --prompt TEXT")
    return args


# ---------------------------------------------------------------------------

class _Text:
    """Text in and out through the folder's tokenizer.json
    (/root/reference/crates/nnis-cli/src/main.rs:1075-1096: special tokens are
    added on encoding and skipped on decoding)."""

    def __init__(self, path: str):
        try:
            from tokenizers import Tokenizer
        except ImportError:
            raise RuntimeError("text prompts need the `tokenizers` package; use --prompt-ids instead") from None
        if not os.path.isfile(path):
            raise RuntimeError(f"tokenizer file {path} does not exist; use --prompt-ids for a model without one")
        self.tokenizer = Tokenizer.from_file(path)

    def encode(self, text: str) -> List[int]:
        ids = self.tokenizer.encode(text, add_special_tokens=True).ids
        if not ids:
            raise RuntimeError("prompt produced no tokens")
        return list(ids)

    def decode(self, ids: List[int]) -> str:
        return self.tokenizer.decode(ids, skip_special_tokens=True)


def run(args: GenerateArgs, out=sys.stdout) -> int:
    from .api import load_engine
    from .engine.generate import GenerationRequest, generate
    from .sampling.params import SamplingParams

    name = "nnis generate-batch" if args.batch else "nnis generate"
    try:
        text = None
        if any(not ids for ids in args.prompt_ids):
            text = _Text(args.tokenizer_file or os.path.join(args.model_dir, "tokenizer.json"))
        prompts = [ids if ids else text.encode(prompt) for prompt, ids in zip(args.prompts, args.prompt_ids)]
        as_ids = [bool(ids) for ids in args.prompt_ids]
        max_tokens = args.max_tokens or sum(((len(p) + args.max_new_tokens + 63) // 64) * 64 for p in prompts)
        engine = load_engine(args.model_dir, dtype=args.dtype, max_tokens=max_tokens, device=f"cuda:{args.device_ordinal}",
                             narrow_to_bfloat16=args.narrow_to_bfloat16)
        stops = engine.model.spec.stop_token_ids  # from the model's metadata (main.rs:1291-1296)

        def show(ids: List[int], ids_out: bool) -> str:
            return ",".join(str(t) for t in ids) if ids_out else text.decode(ids)

        requests = []
        for index, prompt in enumerate(prompts):
            sampling = None
            if args.sample:
                sampling = SamplingParams(seed=args.seeds[index], temperature=args.temperature or 1.0,
                                          top_k=args.top_k, top_p=args.top_p)
            callback = None
            if args.stream:
                def callback(_, token, ids_out=as_ids[index]):
                    out.write((str(token) + " ") if ids_out else text.decode([token]))
                    out.flush()
                    return True
            requests.append(GenerationRequest(prompt, args.max_new_tokens, stops, sampling, callback))
    except Exception as error:  # noqa: BLE001 - every failure becomes the command's error line
        print(f"{name}: {error}", file=sys.stderr)
        return 1

    if not args.batch:
        try:
            result = generate(engine, requests)[0]
        except Exception as error:  # noqa: BLE001
            print(f"{name}: {error}", file=sys.stderr)
            return 1
        if args.stream:
            out.write("\n")
        else:
            out.write(show(result.tokens, as_ids[0]) + "\n")
        return 0

    items = []
    try:
        results = generate(engine, requests)
        for index, result in enumerate(results):
            items.append({"batch_index": index, "seed": args.seeds[index], "ok": True,
                          "text": show(result.tokens, as_ids[index]), "error": None})
    except Exception as error:  # noqa: BLE001
        print(f"{name}: {error}", file=sys.stderr)
        return 1
    if args.json:
        out.write(json.dumps({"schema_version": GENERATE_BATCH_JSON_SCHEMA_VERSION,
                              "sampling_policy_version": SAMPLING_POLICY_VERSION,
                              "session_count": len(items), "results": items}, indent=2) + "\n")
    else:
        out.write(f"NNIS generate-batch sampling_policy_v{SAMPLING_POLICY_VERSION} "
                  f"cli_json_schema_v{GENERATE_BATCH_JSON_SCHEMA_VERSION}\n")
        for item in items:
            out.write(f"=== batch_index {item['batch_index']} seed {item['seed']} ===\n")
            out.write(item["text"] + "\n" if item["ok"] else f"ERROR: {item['error']}\n")
    return 0 if all(item["ok"] for item in items) else 1


def main(argv: Optional[List[str]] = None) -> int:
    try:
        parsed = parse_args(list(sys.argv[1:] if argv is None else argv))
    except UsageError as error:
        print(error, file=sys.stderr)
        return 2
    if parsed == "help":
        print(USAGE)
        return 0
    return run(parsed)


if __name__ == "__main__":
    sys.exit(main())
