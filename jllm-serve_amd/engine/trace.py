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


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64); sizes the page pool")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-live", type=int, default=4, help="most requests live at a time")
    args = ap.parse_args(argv)

    print("trace_run: loading the engine (kernels are compiled on first use)", file=sys.stderr, flush=True)
    from ..kernels import ops
    ops.library()  # compile / load before touching the model, with progress lines on stderr
    from .build import build_runner, load_model
    from .step import StepEntry

    os.makedirs(args.out, exist_ok=True)
    pool_tokens = max(64, -(-args.max_tokens // 64) * 64)
    from ..config import load_config
    # a request can hold at most what the pool holds, even beyond the model's trained length (the reference only
    # warns when the runtime context exceeds max_position_embeddings, cpu/CpuBackend.java:231-234)
    max_positions = max(load_config(args.model).max_positions, pool_tokens)
    model = load_model(args.model, args.dtype, max_positions=max_positions)
    runner = build_runner(model, page_size=args.page_size, pool_tokens=pool_tokens, max_requests=args.max_live,
                          max_positions=max_positions)
    print(f"trace_run: {model.config.description}; {args.dtype}; pool {pool_tokens} tokens in pages of {args.page_size}",
          file=sys.stderr, flush=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        if entries:
            logits = runner.step(entries)
            if logits.shape[0] > 0:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                arr.tofile(os.path.join(args.out, f"{step}.f32"))
        for rid in rec.get("end", []):
            runner.finish(rid)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
