"""Process entry point: one generation request in, one JSON result file out.

    python -m nnis_amd.process --model DIR (--prompt TEXT | --prompt-ids IDS) --result FILE
        [--tokenizer FILE] [--device N] [--max-new-tokens N] [--nnis-bin PATH] [--timeout-seconds S]

The reference offers the same surface around its native binary
(/root/reference/tools/nnis_hub_hf_generate.py:413-423 options, :51-76 request
rules, :109-180 bounded child process, :234-264 a result file that is never
overwritten; contract /root/reference/docs/HF_GENERATION_PROCESS.md:1-60).  Here
the child is this library's ``nnis generate``; decoding is greedy.  The result
records what was asked, what the child printed and how it ended; it claims
nothing about quality or speed.
"""

from __future__ import annotations

import argparse
import hashlib
import json
import os
import subprocess
import sys
import tempfile
import threading
from typing import Any, Dict, List, Optional

SCHEMA_VERSION = 1
CONTRACT = "nnis_amd.generation@1"
MAX_PROMPT_BYTES = 1024 * 1024
MAX_NEW_TOKENS = 65536
MAX_CAPTURE_BYTES = 16 * 1024 * 1024
DEFAULT_TIMEOUT_SECONDS = 3600.0


class RequestError(ValueError):
    pass


def validate_request(model: str, tokenizer: Optional[str], prompt: Optional[str], prompt_ids: Optional[str], device: int,
                     max_new_tokens: int, result: str) -> None:
    if os.path.islink(model) or not os.path.isdir(model):
        raise RequestError(f"--model must name a real folder (symbolic links are refused): {model}")
    if (prompt is None) == (prompt_ids is None):
        raise RequestError("exactly one of --prompt and --prompt-ids is required")
    if prompt is not None:
        if "\0" in prompt:
            raise RequestError("the prompt holds a NUL byte")
        size = len(prompt.encode("utf-8"))
        if not 1 <= size <= MAX_PROMPT_BYTES:
            raise RequestError(f"the prompt is {size} bytes of UTF-8; between 1 and {MAX_PROMPT_BYTES} are taken")
        path = tokenizer or os.path.join(model, "tokenizer.json")
        if os.path.islink(path) or not os.path.isfile(path):
            raise RequestError(f"the tokenizer must be an ordinary file (symbolic links are refused): {path}")
    if not 0 <= device <= 2**31 - 1:
        raise RequestError("--device takes a device number from 0 up")
    if not 1 <= max_new_tokens <= MAX_NEW_TOKENS:
        raise RequestError(f"--max-new-tokens {max_new_tokens} is outside 1 to {MAX_NEW_TOKENS}")
    if os.path.lexists(result):
        raise RequestError(f"result path already exists: {result}")


def run_child(command: List[str], timeout: float, capture_limit: int = MAX_CAPTURE_BYTES) -> Dict[str, Any]:
    """Runs the command without a shell.  Both output channels are drained as
    the child writes them, each by a thread of its own, and never more than
    ``capture_limit`` bytes of a channel are kept: a child that writes more is
    stopped there and the run fails, whatever it would have printed after."""
    try:
        child = subprocess.Popen(command, stdin=subprocess.DEVNULL, stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    except OSError as error:
        return {"status": "not_started", "exit_code": None, "stdout": b"", "stderr": str(error).encode()}
    kept = {"stdout": bytearray(), "stderr": bytearray()}
    over = threading.Event()

    def drain(pipe, name: str) -> None:
        with pipe:
            while True:
                piece = pipe.read1(65536)
                if not piece:
                    return
                room = capture_limit - len(kept[name])
                if len(piece) > room:
                    kept[name] += piece[:room]
                    over.set()
                    child.kill()  # nothing more is wanted from it
                    return
                kept[name] += piece

    readers = [threading.Thread(target=drain, args=(pipe, name), daemon=True)
               for pipe, name in ((child.stdout, "stdout"), (child.stderr, "stderr"))]
    for reader in readers:
        reader.start()
    try:
        code = child.wait(timeout=timeout)
    except subprocess.TimeoutExpired:
        child.kill()
        child.wait()
        for reader in readers:
            reader.join(timeout=5)
        return {"status": "timeout", "exit_code": None, "stdout": b"", "stderr": f"no result within {timeout} s".encode()}
    for reader in readers:
        reader.join(timeout=5)
    if over.is_set():
        return {"status": "output_too_large", "exit_code": code, "stdout": b"",
                "stderr": f"the child wrote more than {capture_limit} bytes to one channel and was stopped".encode()}
    return {"status": "generated" if code == 0 else "failed", "exit_code": code,
            "stdout": bytes(kept["stdout"]), "stderr": bytes(kept["stderr"])}


def build_result(inputs: Dict[str, Any], child: Dict[str, Any]) -> Dict[str, Any]:
    def channel(raw: bytes) -> Dict[str, Any]:
        return {"utf8": raw.decode("utf-8", errors="replace"), "bytes": len(raw), "sha256": hashlib.sha256(raw).hexdigest()}

    return {
        "schema_version": SCHEMA_VERSION,
        "contract": CONTRACT,
        "status": child["status"],
        "exit_code": child["exit_code"],
        "inputs": inputs,
        "sampling": "greedy",
        "stdout": channel(child["stdout"]),
        "stderr": channel(child["stderr"]),
        "network_access": False,
        "serving_performance_verified": False,
        "numerical_equivalence_verified": False,
    }


def write_new_json(path: str, value: Dict[str, Any]) -> None:
    """Writes the whole file, then links it into place: an existing result is never replaced."""
    folder = os.path.dirname(os.path.abspath(path))
    os.makedirs(folder, exist_ok=True)
    encoded = (json.dumps(value, sort_keys=True, separators=(",", ":")) + "\n").encode("utf-8")
    handle = tempfile.NamedTemporaryFile(mode="wb", dir=folder, prefix=".nnis-result-", delete=False)
    try:
        with handle:
            handle.write(encoded)
            handle.flush()
            os.fsync(handle.fileno())
        try:
            os.link(handle.name, path)
        except FileExistsError:
            raise RequestError(f"result path already exists: {path}") from None
    finally:
        try:
            os.unlink(handle.name)
        except OSError:
            pass


def main(argv: Optional[List[str]] = None) -> int:
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    parser = argparse.ArgumentParser(prog="python -m nnis_amd.process", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--model", required=True)
    parser.add_argument("--tokenizer")
    parser.add_argument("--prompt")
    parser.add_argument("--prompt-ids")
    parser.add_argument("--device", type=int, default=0)
    parser.add_argument("--max-new-tokens", type=int, default=16)
    parser.add_argument("--result", required=True)
    parser.add_argument("--nnis-bin", default=os.path.join(here, "bin", "nnis"))
    parser.add_argument("--timeout-seconds", type=float, default=DEFAULT_TIMEOUT_SECONDS)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    args = parser.parse_args(argv)
    try:
        validate_request(args.model, args.tokenizer, args.prompt, args.prompt_ids, args.device, args.max_new_tokens, args.result)
        if not args.timeout_seconds > 0:
            raise RequestError("timeout-seconds must be positive")
    except RequestError as error:
        print(f"nnis_amd.process: {error}", file=sys.stderr)
        return 2
    command = [sys.executable, args.nnis_bin, "generate", "--model", args.model, "--device", str(args.device),
               "--max-new-tokens", str(args.max_new_tokens), "--dtype", args.dtype]
    command += ["--prompt", args.prompt] if args.prompt is not None else ["--prompt-ids", args.prompt_ids]
    if args.tokenizer:
        command += ["--tokenizer", args.tokenizer]
    child = run_child(command, args.timeout_seconds)
    inputs = {"model_directory": args.model, "tokenizer_file": args.tokenizer, "prompt": args.prompt,
              "prompt_ids": args.prompt_ids, "device_ordinal": args.device, "max_new_tokens": args.max_new_tokens,
              "dtype": args.dtype}
    try:
        write_new_json(args.result, build_result(inputs, child))
    except RequestError as error:
        print(f"nnis_amd.process: {error}", file=sys.stderr)
        return 2
    return 0 if child["status"] == "generated" else 1


if __name__ == "__main__":
    sys.exit(main())
