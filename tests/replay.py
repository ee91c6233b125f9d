"""Builds traces for bin/trace_run, runs it, and gathers the logits it wrote."""
import json
import os
import random
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def ceil64(n):
    return -(-n // 64) * 64


class Trace:
    """Steps plus the bookkeeping that says which (request, position) each written row is."""

    def __init__(self, page=64):
        self.page = page  # requests are counted in whole pages of this many tokens
        self.steps = []
        self.rows = {}  # step -> [(rid, position)]
        self.held = {}  # rid -> tokens held
        self.peak = 0

    def add(self, entries, end=()):
        """entries: [(rid, tokens, want)]"""
        n = len(self.steps)
        rec = {"step": n, "entries": [], "end": list(end)}
        rows = []
        for rid, toks, want in entries:
            base = self.held.get(rid, 0)
            rec["entries"].append({"id": rid, "tokens": list(toks), "want": list(want)})
            rows += [(rid, base + w) for w in want]
            self.held[rid] = base + len(toks)
        self.peak = max(self.peak, sum(-(-v // self.page) * self.page for v in self.held.values()))
        for rid in end:
            self.held.pop(rid)
        self.steps.append(rec)
        if rows:
            self.rows[n] = rows
        return n


def whole(trace, rid, toks):
    trace.add([(rid, toks, range(len(toks)))], end=[rid])


def tail_one_by_one(trace, rid, toks, tail=32):
    head = max(1, len(toks) - tail)
    trace.add([(rid, toks[:head], range(head))])
    for i in range(head, len(toks)):
        trace.add([(rid, toks[i:i + 1], [0])], end=[rid] if i == len(toks) - 1 else [])
    if head == len(toks):
        trace.add([], end=[rid])


def portions(trace, rid, toks, sizes=(7, 2, 16, 3, 2, 33, 5, 2, 9)):
    pos, i = 0, 0
    while pos < len(toks):
        n = min(sizes[i % len(sizes)], len(toks) - pos)
        i += 1
        trace.add([(rid, toks[pos:pos + n], range(n))], end=[rid] if pos + n == len(toks) else [])
        pos += n


def mixed(trace, requests, seed=0, live_max=4, decode_tail=8):
    """requests: {rid: tokens}. Up to live_max live; portions of 2..17 tokens of some beside single tokens of
    others; a request is sometimes left out of a step; finished requests are ended so their pages return."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}  # rid -> [tokens, pos]
    while waiting or live:
        while waiting and len(live) < live_max and (not live or rng.random() < 0.7):
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, ended = [], []
        for rid, st in list(live.items()):
            toks, pos = st
            if len(live) > 1 and rng.random() < 0.2:
                continue  # left out of this step
            left = len(toks) - pos
            n = 1 if left <= decode_tail else min(left - decode_tail, rng.choice([2, 2, 3, 5, 8, 13, 17]))
            if left > decode_tail and n == 1:
                n = min(2, left)
            entries.append((rid, toks[pos:pos + n], range(n)))
            st[1] = pos + n
            if st[1] == len(toks):
                ended.append(rid)
                del live[rid]
        if entries or ended:
            trace.add(entries, end=ended)


def run(model_dir, dtype, trace, out_dir, page_size=None, max_tokens=None, timeout=600, env=None, shuffle_free=None):
    """Feeds the trace step by step (the next step only after ``done <step>``) and returns {step: array}."""
    cmd = [sys.executable, TRACE_RUN, "--model", model_dir, "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(max_tokens or trace.peak)]
    if page_size:
        cmd += ["--page-size", str(page_size)]
    if shuffle_free is not None:
        cmd += ["--shuffle-free", str(shuffle_free)]
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for rec in trace.steps:
            p.stdin.write(json.dumps(rec) + "\n")
            p.stdin.flush()
            line = p.stdout.readline()
            assert line.strip() == f"done {rec['step']}", f"trace_run said {line!r} after step {rec['step']}"
        p.stdin.close()
        assert p.wait(timeout=timeout) == 0
    finally:
        if p.poll() is None:
            p.kill()
    out = {}
    for step in trace.rows:
        out[step] = np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4")
    return out
