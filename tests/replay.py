"""Drives bin/trace_run as a user would: writes steps to its standard input,
waits for ``done <step>`` after each, reads the logits files it leaves."""

import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def run_trace(model_dir, dtype, steps, out_dir, max_tokens, vocab, timeout=300):
    """``steps``: list of {"entries": [{"id", "tokens", "want"}], "end": [...]}.
    Returns {(request id, position): logits row}; ``position`` counts the
    request's tokens from its first."""
    process = subprocess.Popen(
        [sys.executable, TRACE_RUN, "--model", model_dir, "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    fed = {}
    rows = {}
    try:
        for number, step in enumerate(steps):
            record = {"step": number, "entries": step["entries"], "end": step.get("end", [])}
            process.stdin.write(json.dumps(record) + "\n")
            process.stdin.flush()
            line = process.stdout.readline().strip()
            if line != f"done {number}":
                process.kill()
                _, err = process.communicate()
                raise AssertionError(f"trace_run answered {line!r} to step {number}\n{err[-3000:]}")
            wanted = [(e["id"], fed.get(e["id"], 0) + w) for e in step["entries"] for w in e.get("want", [])]
            for entry in step["entries"]:
                fed[entry["id"]] = fed.get(entry["id"], 0) + len(entry["tokens"])
            for request in step.get("end", []):
                fed.pop(request, None)
            path = os.path.join(out_dir, f"{number}.f32")
            if wanted:
                data = np.fromfile(path, dtype="<f4")
                assert data.size == len(wanted) * vocab, f"step {number}: {data.size} floats for {len(wanted)} rows"
                for key, row in zip(wanted, data.reshape(len(wanted), vocab)):
                    assert key not in rows, f"{key} asked twice"
                    rows[key] = row
            else:
                assert not os.path.exists(path)
        process.stdin.close()
        assert process.wait(timeout=timeout) == 0, process.stderr.read()[-3000:]
    finally:
        if process.poll() is None:
            process.kill()
    return rows


def whole(requests):
    """Each request alone and whole, one after another."""
    return [{"entries": [{"id": name, "tokens": tokens, "want": list(range(len(tokens)))}], "end": [name]}
            for name, tokens in requests.items()]


def tail_one_by_one(requests, tail=32):
    """A request's first tokens in one step, then its last ``tail`` one by one."""
    steps = []
    for name, tokens in requests.items():
        head = max(1, len(tokens) - tail)
        steps.append({"entries": [{"id": name, "tokens": tokens[:head], "want": list(range(head))}]})
        for index in range(head, len(tokens)):
            steps.append({"entries": [{"id": name, "tokens": [tokens[index]], "want": [0]}],
                          "end": [name] if index == len(tokens) - 1 else []})
        if head == len(tokens):
            steps[-1]["end"] = [name]
    return steps


def unequal_batches(requests, batch, decode):
    """Batches of ``batch`` requests that start together: all but the last
    ``decode`` tokens of each (at least one) in one step, then one token each;
    a request whose tokens run out ends and the others go on."""
    names = list(requests)
    steps = []
    for start in range(0, len(names), batch):
        group = names[start:start + batch]
        heads = {n: max(1, len(requests[n]) - decode) for n in group}
        done = [n for n in group if heads[n] == len(requests[n])]
        steps.append({"entries": [{"id": n, "tokens": requests[n][:heads[n]], "want": list(range(heads[n]))} for n in group],
                      "end": done})
        position = dict(heads)
        live = [n for n in group if n not in done]
        while live:
            entries = [{"id": n, "tokens": [requests[n][position[n]]], "want": [0]} for n in live]
            for n in live:
                position[n] += 1
            done = [n for n in live if position[n] == len(requests[n])]
            steps.append({"entries": entries, "end": done})
            live = [n for n in live if n not in done]
    return steps
