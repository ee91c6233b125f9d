"""Trace replay: feeds given token ids through the model step by step and writes logits.

It drives the same model, step function, cache manager and kernels that generation uses and samples
nothing. Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step that wants logits, ``<out>/<step>.f32`` gets them as little-endian fp32 [wanted, vocab], in the
order of the entries and of ``want``. After every step ``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


class TraceRunner:
    """A model folder opened for replay: ``step(record)`` runs one step of a trace through the engine's step
    function and returns the logits it asked for (or None). ``bin/trace_run`` is a loop around it."""

    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16, max_live: int = 4,
                 shuffle_free=None, model=None):
        """``model``: a model already built (with ``max_positions`` of at least the pool's size), in place of the
        folder."""
        import random

        from ..config import load_config
        from ..kernels import ops
        ops.library()  # compile / load before touching the model, with progress lines on stderr
        from .build import build_runner, load_model
        # the pool holds what the live requests may hold, in whole pages
        self.pool_tokens = max(1, -(-max_tokens // page_size)) * page_size
        if model is None:
            # a request can hold at most what the pool holds, even beyond the model's trained length (the reference
            # only warns when the runtime context exceeds max_position_embeddings, cpu/CpuBackend.java:231-234)
            max_positions = max(load_config(model_dir).max_positions, self.pool_tokens)
            model = load_model(model_dir, dtype, max_positions=max_positions)
        self.model = model
        self.runner = build_runner(model, page_size=page_size, pool_tokens=self.pool_tokens, max_requests=max_live,
                                   max_positions=min(model.build.max_positions, max(model.config.max_positions, self.pool_tokens)))
        self.rng = random.Random(shuffle_free) if shuffle_free is not None else None

    def step(self, rec):
        from .step import StepEntry
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        logits = None
        if entries:
            if self.rng is not None:  # page ids then do not follow positions or the order of requests
                for g in self.runner.cache.groups:
                    g.pool.shuffle_free(self.rng)
            out = self.runner.step(entries)
            if out.shape[0] > 0:
                logits = out
        for rid in rec.get("end", []):
            self.runner.finish(rid)
        return logits


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to whole pages); sizes the page pool")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-live", type=int, default=4, help="most requests live at a time")
    ap.add_argument("--shuffle-free", type=int, default=None, metavar="SEED",
                    help="reorder the free pages before every step (seeded): page ids then follow no pattern")
    args = ap.parse_args(argv)

    print("trace_run: loading the engine (kernels are compiled on first use)", file=sys.stderr, flush=True)
    os.makedirs(args.out, exist_ok=True)
    tr = TraceRunner(args.model, args.dtype, args.max_tokens, args.page_size, args.max_live, args.shuffle_free)
    print(f"trace_run: {tr.model.config.description}; {args.dtype}; pool {tr.pool_tokens} tokens in pages of {args.page_size}",
          file=sys.stderr, flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        logits = tr.step(rec)
        if logits is not None:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            arr.tofile(os.path.join(args.out, f"{rec['step']}.f32"))
        print(f"done {rec['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
