"""The command line, in the reference's manner (Main.java:37-131, :363-390): ``jllm <command> [options]``."""
from __future__ import annotations

import json
import os
import sys

USAGE = """usage: jllm <command> [options]
  run        single completion of a prompt given as token ids (--prompt "1 7 42 ...")
  bench      measure prefill/decode throughput
  config     print the effective configuration and where each value comes from
  random     write a model folder with random weights (--config-json <file> --seed <s> --out <folder>)
options (defaults in jllm.properties; override with --config <file> or flags):
  --model <folder>   --dir <path>   --dtype bfloat16|float32   --ctx <n>   --batch <n>   --page-size <n>   --slots <n>
  --temp <t> --top-k <k> --top-p <p> --min-p <p> --rep-penalty <r> --seed <s> --max-tokens <n> --ignore-eos
  --prompt "<ids>"   --random-weights <seed> (with --config-json <file>: no model folder needed)
  any property key directly, e.g. --backend.kv-pool-tokens 4096 or --bench.rounds=5
not built in this engine: chat, serve, download (no tokenizer, no server, no network)"""


def _fail(msg: str) -> int:
    print(msg, file=sys.stderr)
    return 2


def _prompt_ids(text: str):
    try:
        return [int(t) for t in text.replace(",", " ").split()]
    except ValueError:
        raise ValueError("this engine has no tokenizer: --prompt takes token ids separated by spaces or commas") from None


def build_engine(s):
    """Settings -> Engine (ModelLoader.java:159-210, :658-759)."""
    from .config import load_config, parse_config
    from .engine import Engine, SchedulerConfig
    from .engine.build import build_model, build_runner, parse_dtype, require_gpu
    from .weights import SafetensorsSource
    from .weights.random_init import random_source
    device = require_gpu()
    dtype = parse_dtype(s.get("backend.dtype"))
    if s.has("random-weights"):
        if not s.has("config-json"):
            raise ValueError("--random-weights needs --config-json <file>")
        with open(s.get("config-json")) as f:
            cdict = json.load(f)
        cfg = parse_config(cdict)
        source = random_source(cdict, int(s.get("random-weights")), gain_std=0.0, device=device)
    else:
        if not s.has("model.repo"):
            raise ValueError("no model: pass --model <folder> (or --random-weights <seed> --config-json <file>)")
        path = s.get("model.repo")
        under = os.path.join(s.get("model.dir"), path)
        path = under if not os.path.isabs(path) and os.path.isdir(under) else path
        cfg = load_config(path)
        source = SafetensorsSource(path)
    ctx = s.int_or_auto("backend.ctx") or min(cfg.max_positions, s.get_int("backend.ctx-max"))
    if ctx > cfg.max_positions:
        print(f"warning: context {ctx} exceeds the model's max_position_embeddings {cfg.max_positions}", file=sys.stderr)
    batch = s.int_or_auto("backend.batch") or 2048
    slots = s.get_int("server.slots")
    print(cfg.description, file=sys.stderr)
    model = build_model(cfg, source, dtype, device, ctx)
    runner = build_runner(model, page_size=s.get_int("backend.kv-block"), pool_tokens=s.get_int("backend.kv-pool-tokens"),
                          max_requests=slots, max_positions=ctx, prefix_share=s.get_bool("backend.kv-prefix-share"))
    if runner.cache.sharing_refused:
        print(f"prefix sharing is off: {runner.cache.sharing_refused}", file=sys.stderr)
    budget = s.get_int("engine.pass-budget") or batch + s.get_int("engine.mixed-reserve")
    sc = SchedulerConfig(max_batch_tokens=budget, prefill_chunk=batch, max_running=s.get_int("engine.max-running"),
                         max_positions=ctx, age_promote_s=s.get_int("engine.age-promote-ms") / 1e3,
                         session_max_running=s.get_int("engine.session-max-running"),
                         background_chunk_cap=s.get_int("engine.background-chunk-cap"), preempt=s.get_bool("engine.preempt"))
    import torch
    props = torch.cuda.get_device_properties(device)
    print(f"backend: HIP kernels on {props.name} ({props.multi_processor_count} compute units), {s.get('backend.dtype')}, ctx {ctx}, batch {batch}, {slots} slots, "
          f"KV pool {runner.cache.num_pages} pages of {runner.cache.page_size}", file=sys.stderr)
    return Engine(runner, sc, eos_token_ids=cfg.eos_token_ids)


def stats_line(st) -> str:
    return (f"{int(st.get('prompt_tokens', 0))} prompt tok ({int(st.get('cached_tokens', 0))} cached), prefill {st.get('prefill_ms', 0):.0f} ms, "
            f"{int(st.get('generated_tokens', 0))} generated in {st.get('decode_ms', 0):.0f} ms = {st.get('tok_per_sec', 0):.1f} tok/s")


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] in ("-h", "--help", "help"):
        print(USAGE, file=sys.stderr)
        return 0 if argv else 2
    from .config.settings import Settings, SettingsError
    cmd = argv[0]
    try:
        s = Settings.load(argv).validate()
    except SettingsError as e:
        return _fail(str(e))
    if cmd == "config":
        for k, v, src in s.describe():
            print(f"{k}={v}    [{src}]")
        return 0
    if cmd == "random":
        from .weights import write_random_model
        if not (s.has("config-json") and s.has("out")):
            return _fail("random needs --config-json <file> and --out <folder>")
        with open(s.get("config-json")) as f:
            cdict = json.load(f)
        seed = s.get_int("sampling.seed")
        print(write_random_model(s.get("out"), cdict, max(seed, 0)))
        return 0
    if cmd in ("chat", "serve", "download", "image", "video", "transcribe", "speak"):
        return _fail(f"'{cmd}' is not part of this engine (token ids in, token ids out; see 'run')")
    if cmd not in ("run", "bench"):
        print(USAGE, file=sys.stderr)
        return 2
    try:
        engine = build_engine(s)
    except (ValueError, OSError, RuntimeError) as e:  # a bad folder or option, no GPU, a kernel library that will not build
        return _fail(str(e))
    if cmd == "run":
        try:
            prompt = _prompt_ids(s.get("prompt")) if s.has("prompt") else [1]
        except ValueError as e:
            return _fail(str(e))
        if not s.get_bool("json"):
            engine.on_token = lambda rid, tok: print(tok, end=" ", flush=True)
        r = engine.generate([prompt], s.sampling())[0]
        if s.get_bool("json"):
            print(json.dumps({"tokens": r.tokens, "finish_reason": r.finish_reason}))
        else:
            print()
        print(stats_line(r.stats) + f", finish={r.finish_reason}", file=sys.stderr)
        return 0
    # bench (Main.java:363-382): a warm-up, then rounds of prefill + decode of the same prompt
    pattern = [11, 23, 5, 42, 7, 19, 3, 31, 13, 2]
    vocab = engine.runner.vocab
    prompt = [t % vocab for t in pattern] * s.get_int("bench.prompt-repeat")
    p = s.sampling().with_max_tokens(s.get_int("bench.max-tokens"))
    from dataclasses import replace
    p = replace(p, ignore_eos=True)
    engine.generate([prompt], p)
    for _ in range(s.get_int("bench.rounds")):
        engine.runner.cache.drop_cached()  # every round prefills the whole prompt (Main.java:372-373 evicts the prefix with another prompt)
        st = engine.generate([prompt], p)[0].stats
        pt, g = st["prompt_tokens"] - st.get("cached_tokens", 0), st["generated_tokens"]
        print(f"prefill {int(pt)} tok in {st['prefill_ms']:.0f} ms ({pt / (st['prefill_ms'] / 1e3):.1f} tok/s), "
              f"decode {int(g)} tok in {st['decode_ms']:.0f} ms ({st['tok_per_sec']:.1f} tok/s)")
    return 0


if __name__ == "__main__":
    sys.exit(main())
