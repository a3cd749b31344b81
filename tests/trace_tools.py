"""Traces in the format of bin/trace_run, the ways to cut requests into steps, and a runner."""
from __future__ import annotations

import json
import os
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def round64(n: int) -> int:
    return -(-n // 64) * 64


def whole(requests: dict) -> list[dict]:
    """Each request alone and whole."""
    return [{"step": i, "entries": [{"id": rid, "tokens": ids, "want": list(range(len(ids)))}], "end": [rid]}
            for i, (rid, ids) in enumerate(requests.items())]


def decode_tail(requests: dict, tail: int = 32) -> list[dict]:
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps = []
    for rid, ids in requests.items():
        head = max(1, len(ids) - tail)
        cuts = [0, head] + list(range(head + 1, len(ids) + 1))
        for a, b in zip(cuts, cuts[1:]):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": ids[a:b], "want": list(range(b - a))}],
                          "end": [rid] if b == len(ids) else []})
    return steps


def portions(requests: dict, seed: int) -> list[dict]:
    """Portions of changing size, down to two tokens (and one at the very end if it comes out so)."""
    rng = np.random.default_rng(seed)
    steps = []
    for rid, ids in requests.items():
        at = 0
        while at < len(ids):
            size = int(rng.choice([2, 3, 5, 16, 17, 31, 33, 64]))
            size = min(size, len(ids) - at)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": ids[at:at + size],
                                                          "want": list(range(size))}],
                          "end": [rid] if at + size == len(ids) else []})
            at += size
    return steps


def mixed(requests: dict, seed: int, max_live: int = 4, tail: int = 12) -> list[dict]:
    """Up to `max_live` requests at a time: portions of some beside single tokens of others; a request may
    sit out a step.  The last `tail` tokens of each request come one by one, as decoding does."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live: dict = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, ids = waiting.pop(0)
            live[rid] = [ids, 0]
        entries, ended = [], []
        for rid, state in live.items():
            ids, at = state
            if len(live) > 1 and rng.random() < 0.25:
                continue
            left = len(ids) - at
            size = 1 if left <= tail else min(int(rng.choice([2, 3, 7, 16, 29, 40])), left - tail)
            entries.append({"id": rid, "tokens": ids[at:at + size], "want": list(range(size))})
            state[1] = at + size
            if state[1] == len(ids):
                ended.append(rid)
        if not entries:
            continue
        for rid in ended:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def peak_tokens(steps: list[dict]) -> int:
    """Most tokens live requests hold at any time, each rounded up to 64."""
    held: dict = {}
    peak = 0
    for step in steps:
        for entry in step["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        peak = max(peak, sum(round64(n) for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return peak


def run_in_process(engine, steps: list[dict]) -> dict:
    """Run a trace on an engine; returns {request id: logits [its tokens, vocab]} (float32, CPU)."""
    from tokenizer_amd.engine import StepEntry
    out: dict = {}
    for step in steps:
        entries = []
        for item in step["entries"]:
            if not engine.has_request(item["id"]):
                engine.add_request(item["id"])
            entries.append(StepEntry(item["id"], item["tokens"], item["want"]))
        logits = engine.step(entries).float().cpu()
        row = 0
        for item in step["entries"]:
            n = len(item["want"])
            out.setdefault(item["id"], []).append(logits[row:row + n])
            row += n
        for rid in step["end"]:
            engine.end_request(rid)
    return {rid: torch.cat(parts) for rid, parts in out.items()}


def run_program(model_folder: str, dtype: str, steps: list[dict], out_dir: str, max_tokens: int, vocab: int,
                env: dict | None = None) -> dict:
    """Run a trace through bin/trace_run as a child process, step by step, waiting for each `done`."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folder, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {step['step']}", f"expected 'done {step['step']}', got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    out: dict = {}
    for step in steps:
        wanted = sum(len(e["want"]) for e in step["entries"])
        if not wanted:
            continue
        data = np.fromfile(os.path.join(out_dir, f"{step['step']}.f32"), dtype="<f4").reshape(wanted, vocab)
        row = 0
        for item in step["entries"]:
            n = len(item["want"])
            out.setdefault(item["id"], []).append(torch.from_numpy(data[row:row + n].copy()))
            row += n
    return {rid: torch.cat(parts) for rid, parts in out.items()}
