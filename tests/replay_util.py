"""Builds replay traces (the ways of cutting and batching requests) and drives bin/trace_run."""
import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent


class Trace:
    """Steps for trace_run plus, per step, which (request, position) each output row is."""

    def __init__(self):
        self.steps = []
        self.rows = {}      # step -> [(request name, position)]
        self.fed = {}       # request name -> tokens fed so far

    def step(self, entries, end=()):
        """entries: [(name, tokens, want)]"""
        idx = len(self.steps)
        rows = []
        recs = []
        for name, tokens, want in entries:
            base = self.fed.get(name, 0)
            recs.append({"id": name, "tokens": [int(t) for t in tokens], "want": [int(w) for w in want]})
            rows += [(name, base + int(w)) for w in want]
            self.fed[name] = base + len(tokens)
        self.steps.append({"step": idx, "entries": recs, "end": list(end)})
        if rows:
            self.rows[idx] = rows
        for name in end:
            self.fed.pop(name, None)
        return idx


def whole(trace, name, tokens):
    trace.step([(name, tokens, range(len(tokens)))], end=[name])


def tail_one_by_one(trace, name, tokens, tail=32):
    head = len(tokens) - tail
    assert head >= 1
    trace.step([(name, tokens[:head], [head - 1])])
    for i in range(head, len(tokens)):
        trace.step([(name, tokens[i:i + 1], [0])], end=[name] if i == len(tokens) - 1 else [])


def portions(trace, name, tokens, sizes):
    at, i = 0, 0
    while at < len(tokens):
        n = min(sizes[i % len(sizes)], len(tokens) - at)
        last = at + n == len(tokens)
        trace.step([(name, tokens[at:at + n], range(n))], end=[name] if last else [])
        at += n
        i += 1


def mixed(trace, requests, rng, max_live=4, sizes=(2, 5, 9, 16, 23, 3, 31), decode_tail=12):
    """Up to ``max_live`` requests at once: each is fed in portions of changing size and its
    last ``decode_tail`` tokens one by one; every step advances a random subset of the live
    requests (so some sit a step out) and new requests start as others end."""
    pending = list(requests.items())
    live = {}   # name -> [tokens, at]
    k = 0
    peak = 0
    while pending or live:
        while pending and len(live) < max_live:
            name, toks = pending.pop(0)
            live[name] = [toks, 0]
        names = list(live)
        chosen = [n for n in names if rng.random() < 0.75] or [names[int(rng.integers(len(names)))]]
        entries, ended = [], []
        for name in chosen:
            toks, at = live[name]
            left = len(toks) - at
            n = 1 if left <= decode_tail else min(sizes[k % len(sizes)], left - decode_tail)
            k += 1
            entries.append((name, toks[at:at + n], range(n)))
            live[name][1] = at + n
            if at + n == len(toks):
                ended.append(name)
        held = sum(-(-max(s[1], 1) // 64) * 64 for s in live.values())
        peak = max(peak, held)
        trace.step(entries, end=ended)
        for name in ended:
            del live[name]
    return peak


def run_trace(model_dir, dtype, trace, max_tokens, out_dir, block_size=None, timeout=600):
    """Feeds the trace to bin/trace_run one step at a time; returns {step: array [rows, vocab]}."""
    cmd = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
           "--out", str(out_dir), "--max-tokens", str(max_tokens)]
    if block_size:
        cmd += ["--block-size", str(block_size)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, cwd=str(ROOT))
    try:
        for st in trace.steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {st['step']}", f"trace_run said {line!r} at step {st['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=timeout) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    vocab = json.loads((Path(model_dir) / "config.json").read_text())["vocab_size"]
    out = {}
    for idx, rows in trace.rows.items():
        a = np.fromfile(Path(out_dir) / f"{idx}.f32", dtype="<f4")
        assert a.size == len(rows) * vocab, f"step {idx}: {a.size} floats for {len(rows)} rows"
        out[idx] = a.reshape(len(rows), vocab)
    return out


def compare(trace, got, expected, check):
    """``expected``: name -> [T, vocab] array of the plain implementation; ``check(name, pos, got_row,
    want_row)`` is called for every row."""
    n = 0
    for idx, rows in trace.rows.items():
        for r, (name, pos) in enumerate(rows):
            check(name, pos, got[idx][r], expected[name.split("#")[0]][pos])
            n += 1
    return n
