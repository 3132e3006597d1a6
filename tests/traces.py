"""Trace families for the replay program and the driver that talks to it.

A plan is a list of steps ``{"step", "entries": [{"id", "tokens", "want"}], "end"}``; every fed
token's logits are wanted, so a replay yields one row per token, which ``collect`` sorts
back into per-request [length, vocab] arrays for comparison with the plain model.
"""
import json
import os
import random
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def _entry(request, tokens, start, count):
    return {"id": request, "tokens": tokens[start:start + count], "want": list(range(count))}


def whole(requests):
    """Each request alone and whole: one step per request."""
    return [{"entries": [_entry(name, tokens, 0, len(tokens))], "end": [name]} for name, tokens in requests.items()]


def tail_decoded(requests, tail=32):
    """Most of it in one step, the last ``tail`` tokens one by one."""
    steps = []
    for name, tokens in requests.items():
        head = max(1, len(tokens) - tail)
        steps.append({"entries": [_entry(name, tokens, 0, head)], "end": []})
        for position in range(head, len(tokens)):
            steps.append({"entries": [_entry(name, tokens, position, 1)],
                          "end": [name] if position == len(tokens) - 1 else []})
    return steps


def portions(requests, sizes=(7, 2, 5, 3, 11, 2, 1, 13, 2, 4)):
    """Portions of changing size, down to two tokens (and one)."""
    steps = []
    for name, tokens in requests.items():
        cursor, turn = 0, 0
        while cursor < len(tokens):
            count = min(sizes[turn % len(sizes)], len(tokens) - cursor)
            steps.append({"entries": [_entry(name, tokens, cursor, count)],
                          "end": [name] if cursor + count == len(tokens) else []})
            cursor += count
            turn += 1
    return steps


def mixed(requests, seed, live_limit=4, prefill=(9, 2, 17, 5)):
    """Up to ``live_limit`` live requests: portions of some beside single decoded tokens of
    others; a request may sit out a step; finished requests end and the next one starts, so
    with a small pool its pages and slot are used again."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}                  # name -> [tokens, cursor, prompt_length, turn]
    steps = []
    while waiting or live:
        while waiting and len(live) < live_limit:
            name, tokens = waiting.pop(0)
            live[name] = [tokens, 0, max(1, len(tokens) - rng.randint(8, 40)), 0]
        entries, ended = [], []
        for name, state in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                  # left out of this step, goes on later
            tokens, cursor, prompt, turn = state
            if cursor < prompt:
                count = min(prefill[turn % len(prefill)], prompt - cursor)
            else:
                count = 1
            entries.append(_entry(name, tokens, cursor, count))
            state[1] += count
            state[3] += 1
            if state[1] == len(tokens):
                ended.append(name)
                del live[name]
        if entries:
            steps.append({"entries": entries, "end": ended})
    return steps


def number(steps, first=0):
    for index, step in enumerate(steps):
        step["step"] = first + index
    return steps


def peak_tokens(steps, granule=64):
    """The most tokens live requests hold at any time, each rounded up to ``granule``."""
    held, peak = {}, 0
    for step in steps:
        for entry in step["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        peak = max(peak, sum(-(-count // granule) * granule for count in held.values()))
        for name in step["end"]:
            held.pop(name, None)
    return peak


def replay(model_dir, dtype, steps, max_tokens, out_dir, extra=(), timeout=600):
    """Run bin/trace_run, one step at a time: write a line, wait for its ``done``."""
    os.makedirs(out_dir, exist_ok=True)
    command = [sys.executable, TRACE_RUN, "--model", str(model_dir), "--dtype", dtype, "--out", str(out_dir),
               "--max-tokens", str(max_tokens)] + list(extra)
    process = subprocess.Popen(command, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, cwd=str(out_dir))
    try:
        for step in steps:
            process.stdin.write(json.dumps(step) + "\n")
            process.stdin.flush()
            line = process.stdout.readline()
            if line.strip() != f"done {step['step']}":
                raise AssertionError(f"trace_run answered {line!r} to step {step['step']} "
                                     f"(exit code {process.poll()})")
        process.stdin.close()
        code = process.wait(timeout=timeout)
    finally:
        if process.poll() is None:
            process.kill()
    assert code == 0, f"trace_run exited with {code}"


def collect(steps, out_dir, vocab, lengths):
    """name -> float32 [length, vocab] from the <step>.f32 files."""
    out = {name: np.full((length, vocab), np.nan, dtype=np.float32) for name, length in lengths.items()}
    cursor = {name: 0 for name in lengths}
    for step in steps:
        wanted = sum(len(entry["want"]) for entry in step["entries"])
        path = os.path.join(str(out_dir), f"{step['step']}.f32")
        if wanted == 0:
            assert not os.path.exists(path)
        else:
            rows = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
        row = 0
        for entry in step["entries"]:
            for place in entry["want"]:
                out[entry["id"]][cursor[entry["id"]] + place] = rows[row]
                row += 1
            cursor[entry["id"]] += len(entry["tokens"])
    return out
