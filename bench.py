"""Decode and prefill throughput of the engine at the Qwen3-8B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch through the engine's own loop (scheduler, step function, paged
cache, kernels, device-side selection). Prints one JSON line. Peaks used for the fractions are the published
MI355X figures: HBM 8 TB/s; dense MFMA 2.5 PFLOP/s for bf16, 157.3 TFLOP/s for fp32. Beside them the line gives the
same fractions against what this GPU delivered to two probes run at the start (a kernel that only streams memory
in, a kernel that only issues bf16 MFMAs): `frac_measured`.

The default run also reports, under `points` (flat, every figure with the bytes or flops fraction behind it):
decoding at batch 1 and 64; decoding at the context lengths the configurations name (batch 8 near 8,192 keys, batch
64 near 4,096); a sampled decode step (temperature, top-k, top-p on the device); the prefill of one 8,192-token
prompt in portions of 2,048; the float32 path of the same shape on fewer layers (`config` names both counts);
steady decoding at the 14B and 32B shapes (the 32B shape also with 16,000 keys per request); and the 14B and 32B
request sets served to the end, with the time the roofline allows for their passes as a fraction of the time taken.
`--no-serve`, `--no-fp32`, `--no-long` and `--no-shapes` leave groups out; `--temperature/--top-k/--top-p` make the
main decode run a sampled one.

A decode step must read every weight once and the keys and values of the live requests: bytes = weights + KV bytes
per token x tokens held (mean over the timed steps). A prefill must do 2 flops per weight and row, plus 4 x heads x
head size per (row, key) pair and layer, plus the head for the rows whose logits are wanted.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
PAGE = 16

SHAPES = {  # Qwen3 dense layer sizes: (layers, hidden, heads, kv heads, head dim, intermediate, context)
    "0.6b": (28, 1024, 16, 8, 128, 3072, 8192),
    "1.7b": (28, 2048, 16, 8, 128, 6144, 8192),
    "4b": (36, 2560, 32, 8, 128, 9728, 8192),
    "8b": (36, 4096, 32, 8, 128, 12288, 8192),
    "14b": (40, 5120, 40, 8, 128, 17408, 8192),
    "32b": (64, 5120, 64, 8, 128, 25600, 16384),
}


def shape_config(name="8b"):
    """A config.json of a Qwen3 dense model's layer sizes (untied output head, as in the larger ones)."""
    L, d, H, Hkv, hd, F, ctx = SHAPES[name]
    return dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=L, hidden_size=d,
                num_attention_heads=H, num_key_value_heads=Hkv, head_dim=hd, intermediate_size=F,
                vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False,
                max_position_embeddings=ctx)


class Work:
    """Bytes and flops that passes over a model of these sizes must move (the roofline's numerators)."""

    def __init__(self, shape: dict, dtype: str):
        self.L, self.d = shape["num_hidden_layers"], shape["hidden_size"]
        self.H, self.Hkv, self.hd = shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
        self.F, self.V = shape["intermediate_size"], shape["vocab_size"]
        self.esize = 2 if dtype == "bf16" else 4
        self.dtype = dtype
        self.layer_params = (self.H * self.hd + 2 * self.Hkv * self.hd) * self.d + self.d * self.H * self.hd + 3 * self.d * self.F
        self.weight_bytes = (self.L * self.layer_params + self.V * self.d) * self.esize
        self.kv_bytes_per_token = 2 * self.L * self.Hkv * self.hd * self.esize

    def decode_bytes(self, tokens_held: float) -> float:
        return self.weight_bytes + self.kv_bytes_per_token * tokens_held

    def flops(self, rows: float, pairs: float, selected: float) -> float:
        """``rows`` through every layer, ``pairs`` of (row, key) in the attention of every layer, ``selected`` rows
        through the head."""
        return 2.0 * rows * self.L * self.layer_params + 4.0 * self.H * self.hd * self.L * pairs + 2.0 * self.V * self.d * selected

    def pass_seconds(self, ones: int, one_keys: int, rows: int, pairs: int) -> float:
        """The least time one pass can take at the published peaks: the larger of the time to read what it must
        read (every weight once, the keys and values of the requests that bring one row; the portions' own reads
        are left out) and the time to do its flops."""
        by = self.weight_bytes + self.kv_bytes_per_token * one_keys
        fl = self.flops(ones + rows, one_keys + pairs, ones + (1 if rows else 0))
        return max(by / HBM_PEAK, fl / FLOP_PEAK[self.dtype])


def sampling_of(args, max_tokens: int):
    from jllm_serve_amd.sampling import SamplingParams
    if args.temperature > 0:
        return SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, seed=1,
                              max_tokens=max_tokens, ignore_eos=True)
    return SamplingParams.greedy_params(max_tokens=max_tokens, ignore_eos=True)


def serve_workload(args) -> dict:
    """The 14B and 32B workloads: a set of requests served to the end by the engine (scheduler, mixed passes,
    paged cache near full). 14b: 32 requests, prompts uniform in 128..4096, 128 generated each. 32b: 64 prompts of
    1,024 tokens, 256 generated each, pool of exactly 64 x 1,280 positions. ``roofline_frac``: the sum over the
    passes of the least time each can take at the published peaks (``Work.pass_seconds``), over the wall time."""
    import random

    import torch
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_model, build_runner
    from jllm_serve_amd.kernels import ops
    from jllm_serve_amd.weights.random_init import random_source

    ops.library()
    dev = torch.device("cuda:0")
    shape = shape_config(args.shape)
    if args.layers:
        shape["num_hidden_layers"] = args.layers
    cfg = parse_config(shape)
    ctx = SHAPES[args.shape][6]
    rng = random.Random(0)
    if args.shape == "32b":
        n_req, gen = 64, 256
        lens = [1024] * n_req
        pool = n_req * (1024 + gen)
    else:
        n_req, gen = 32, 128
        lens = [rng.randint(128, 4096) for _ in range(n_req)]
        pool = sum(-(-(n + gen) // 64) * 64 for n in lens)
    V = shape["vocab_size"]
    prompts = [[rng.randrange(V) for _ in range(n)] for n in lens]
    if args.shared_prefix:  # a system prompt in front of every request; the cache shares its pages
        stem = [rng.randrange(V) for _ in range(args.shared_prefix)]
        prompts = [stem[:len(p) - 1] + p[min(len(stem), len(p) - 1):] for p in prompts]
    t0 = time.time()
    model = build_model(cfg, random_source(shape, seed=0, gain_std=0.0, device=dev), "bfloat16" if args.dtype == "bf16" else "float32",
                        dev, ctx)
    runner = build_runner(model, page_size=PAGE, pool_tokens=pool, max_requests=n_req, max_positions=ctx,
                          prefix_share=args.shared_prefix > 0)
    torch.cuda.synchronize()
    print(f"[bench] model built in {time.time() - t0:.0f} s: {cfg.description}", file=sys.stderr, flush=True)
    params = sampling_of(args, gen)

    def run():
        runner.cache.drop_cached()  # nothing of an earlier run is found again
        eng = Engine(runner, SchedulerConfig(max_batch_tokens=args.budget, prefill_chunk=args.budget, max_running=n_req, max_positions=ctx))
        eng.scheduler.ledger = []
        torch.cuda.synchronize()
        t = time.perf_counter()
        res = eng.generate(prompts, params)
        torch.cuda.synchronize()
        return time.perf_counter() - t, res, eng

    run()  # warm-up: captures the decode graphs
    dt, res, eng = run()
    generated = sum(len(r.tokens) for r in res)
    assert generated == n_req * gen
    st = eng.stats()
    work = Work(shape, args.dtype)
    ledger = eng.scheduler.ledger
    ideal = sum(work.pass_seconds(*p) for p in ledger)
    decode_bytes = sum(work.decode_bytes(p[1]) for p in ledger if p[0])
    prompt_flops = sum(work.flops(p[2], p[3], 1 if p[2] else 0) for p in ledger)
    out = {
        "metric": f"generated tok/s serving {n_req} requests to the end (Qwen3-{args.shape.upper()} shape, 1 GPU)",
        "value": round(generated / dt, 2), "unit": "tok/s", "n_gpus": 1, "steps": st["scheduler"]["passes"], "warmup": 1,
        "ms_per_step": round(dt * 1e3 / st["scheduler"]["passes"], 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": f"Qwen3-{args.shape.upper()} shape", "layers": cfg.num_layers, "layers_in_shape": SHAPES[args.shape][0],
                   "hidden": cfg.hidden, "heads": shape["num_attention_heads"], "kv_heads": shape["num_key_value_heads"],
                   "head_dim": shape["head_dim"], "intermediate": shape["intermediate_size"], "vocab": V,
                   "requests": n_req, "prompt_tokens": sum(lens), "generated_per_request": gen, "context": ctx,
                   "pool_tokens": pool, "page_size": PAGE, "pass_budget": args.budget, "shared_prefix": args.shared_prefix, "global_batch": n_req, "seq_len": max(lens), "parallelism": "single GPU"},
        "wall_s": round(dt, 3), "prompt_tok_per_s": round(sum(lens) / dt, 1), "preemptions": st["scheduler"]["preemptions"],
        "rows_per_pass": round(st["scheduler"]["rows_per_pass"], 1),
        "cached_prompt_tokens": int(sum(r.stats.get("cached_tokens", 0) for r in res)),
        "roofline": {"bound": "hbm for the passes that decode, mfma for the portions of prompts", "ideal_s": round(ideal, 4),
                     "frac": round(ideal / dt, 4), "decode_GB": round(decode_bytes / 1e9, 1),
                     "prompt_TFLOP": round(prompt_flops / 1e12, 1), "passes": len(ledger),
                     "passes_with_decoding": sum(1 for p in ledger if p[0])},
    }
    del eng, runner, model
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--context", type=int, default=0, help="positions a request may hold (0: the shape's own)")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--points", default="1,64", help="other decode batch sizes to report")
    ap.add_argument("--point-steps", type=int, default=24)
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="8b is the default run; 14b and 32b with --workload serve")
    ap.add_argument("--budget", type=int, default=8192, help="serve: rows per pass (prompt portions + decoding requests)")
    ap.add_argument("--shared-prefix", type=int, default=0,
                    help="serve: every prompt starts with the same N tokens and the cache shares their pages (0 = off)")
    ap.add_argument("--temperature", type=float, default=0.0, help="sampled decoding in the main run (0: greedy)")
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--no-serve", action="store_true", help="steady: leave out the 14B and 32B request sets")
    ap.add_argument("--no-fp32", action="store_true", help="steady: leave out the float32 figures")
    ap.add_argument("--no-long", action="store_true", help="steady: leave out the long-context and sampled points")
    ap.add_argument("--no-shapes", action="store_true", help="steady: leave out steady decoding at the 14B and 32B shapes")
    ap.add_argument("--fp32-layers", type=int, default=4, help="layers of the float32 run (named in config)")
    ap.add_argument("--workload", default="steady", choices=["steady", "serve"],
                    help="steady: timed decode steps at a fixed batch (the default run); serve: a request set run to the end")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    if args.workload == "serve":
        print(json.dumps(serve_workload(args)))
        return 0

    import torch
    from jllm_serve_amd.kernels import ops

    ops.library()
    torch.cuda.set_device(0)
    peaks = ops.measured_peaks()
    print(f"[bench] measured: HBM read {peaks['hbm_read_bytes_per_s'] / 1e12:.2f} TB/s, bf16 MFMA "
          f"{peaks['mfma_bf16_flop_per_s'] / 1e15:.2f} PFLOP/s", file=sys.stderr, flush=True)
    hbm_meas = peaks["hbm_read_bytes_per_s"]
    flop_meas = peaks["mfma_bf16_flop_per_s"] if args.dtype == "bf16" else None
    context = args.context or SHAPES[args.shape][6]
    full = args.dtype == "bf16" and not args.layers and args.shape == "8b"
    points_b = sorted({int(p) for p in args.points.split(",") if p} | {args.batch})
    decodes = [dict(key=f"b{B}", batch=B, prompt_len=args.prompt_len, steps=args.steps if B == args.batch else args.point_steps,
                    warmup=args.warmup if B == args.batch else 4, sampling=sampling_of(args, 1) if B == args.batch else None)
               for B in points_b]
    prefills = [dict(key="main", tokens=2048, portion=2048)]
    if full and not args.no_long:
        near = context - 64 - args.point_steps - 8  # as many keys as the context allows while the timed steps run
        decodes.append(dict(key="b8_ctx8k", batch=8, prompt_len=near, steps=args.point_steps, warmup=4))
        decodes.append(dict(key="b64_ctx4k", batch=64, prompt_len=context // 2 - 128, steps=args.point_steps, warmup=4))
        sampled = argparse.Namespace(temperature=0.7, top_k=20, top_p=0.95)
        decodes.append(dict(key="b8_sampled", batch=8, prompt_len=args.prompt_len, steps=args.point_steps, warmup=4,
                            sampling=sampling_of(sampled, 1)))
        prefills.append(dict(key="8k", tokens=context, portion=2048))
        prefills.append(dict(key="512", tokens=512, portion=512))
    main_run = steady(args, args.shape, args.dtype, args.layers, context, decodes, prefills)
    step_s, mean_ctx, bytes_step = main_run["decode"][f"b{args.batch}"]
    achieved = bytes_step / step_s
    prefill = dict(main_run["prefill"]["main"])
    if flop_meas:
        prefill["frac_measured"] = round(prefill["flops"] / (prefill["ms"] * 1e-3) / flop_meas, 4)
    prefill.pop("flops")
    points = {}

    def decode_point(name, run, key, B, measured=True):
        s_, ctx_, by = run["decode"][key]
        points[name] = round(B / s_, 2)
        points[name + "_ms"] = round(s_ * 1e3, 3)
        points[name + "_keys"] = int(ctx_ / B)
        points[name + "_hbm_frac"] = round(by / s_ / HBM_PEAK, 4)
        if measured:
            points[name + "_hbm_frac_measured"] = round(by / s_ / hbm_meas, 4)

    for B in points_b:
        if B != args.batch:
            decode_point(f"decode_b{B}", main_run, f"b{B}", B)
    for key, B in (("b8_ctx8k", 8), ("b64_ctx4k", 64), ("b8_sampled", 8)):
        if key in main_run["decode"]:
            decode_point("decode_" + key, main_run, key, B, measured=False)
    if "8k" in main_run["prefill"]:
        p8 = main_run["prefill"]["8k"]
        points["prefill_8k_tok_s"], points["prefill_8k_ms"], points["prefill_8k_frac"] = p8["value"], p8["ms"], p8["frac"]
    if "512" in main_run["prefill"]:
        p5 = main_run["prefill"]["512"]
        points["prefill_512_ms"], points["prefill_512_frac"] = p5["ms"], p5["frac"]
    cfg = dict(main_run["config"])
    if not args.no_fp32 and args.dtype == "bf16":
        f32 = steady(args, args.shape, "fp32", args.fp32_layers, context,
                     [dict(key="b", batch=args.batch, prompt_len=args.prompt_len, steps=max(8, args.steps // 4), warmup=2)],
                     [dict(key="main", tokens=2048, portion=2048)])
        fs, _, fby = f32["decode"]["b"]
        points["fp32_prefill_tok_s"] = f32["prefill"]["main"]["value"]
        points["fp32_prefill_frac"] = f32["prefill"]["main"]["frac"]
        points[f"fp32_decode_b{args.batch}"] = round(args.batch / fs, 2)
        points[f"fp32_decode_b{args.batch}_hbm_frac"] = round(fby / fs / HBM_PEAK, 4)
        cfg["fp32_layers"] = f32["config"]["layers"]
    if full and not args.no_shapes:
        r14 = steady(args, "14b", "bf16", 0, SHAPES["14b"][6],
                     [dict(key="b8", batch=8, prompt_len=2048, steps=args.point_steps, warmup=4),
                      dict(key="b32", batch=32, prompt_len=2048, steps=args.point_steps, warmup=4)], [])
        decode_point("14b_decode_b8", r14, "b8", 8, measured=False)
        decode_point("14b_decode_b32", r14, "b32", 32, measured=False)
        r32 = steady(args, "32b", "bf16", 0, SHAPES["32b"][6],
                     [dict(key="b64", batch=64, prompt_len=1152 - 64, steps=args.point_steps, warmup=4),
                      dict(key="b4_16k", batch=4, prompt_len=16000, steps=args.point_steps, warmup=4)], [])
        decode_point("32b_decode_b64", r32, "b64", 64, measured=False)
        decode_point("32b_decode_b4_ctx16k", r32, "b4_16k", 4, measured=False)
    if not args.no_serve and full:
        for shape in ("14b", "32b"):
            sargs = argparse.Namespace(**{**vars(args), "shape": shape, "layers": 0, "shared_prefix": 0, "temperature": 0.0})
            r = serve_workload(sargs)
            points[f"serve_{shape}_tok_s"] = r["value"]
            points[f"serve_{shape}_prompt_tok_s"] = r["prompt_tok_per_s"]
            points[f"serve_{shape}_wall_s"] = r["wall_s"]
            points[f"serve_{shape}_preemptions"] = r["preemptions"]
            points[f"serve_{shape}_roofline_s"] = r["roofline"]["ideal_s"]
            points[f"serve_{shape}_roofline_frac"] = r["roofline"]["frac"]
            points[f"serve_{shape}_decode_GB"] = r["roofline"]["decode_GB"]
            points[f"serve_{shape}_prompt_TFLOP"] = r["roofline"]["prompt_TFLOP"]
            print(f"[bench] serve {shape}: {r['value']} generated tok/s, {r['wall_s']} s, the roofline allows "
                  f"{r['roofline']['ideal_s']} s", file=sys.stderr, flush=True)
    sampled_main = args.temperature > 0
    out = {
        "metric": ("decode tok/s at batch 8 (Qwen3-8B shape, 1 GPU)" if args.batch == 8 and args.shape == "8b" else
                   f"decode tok/s at batch {args.batch}") + (" sampled" if sampled_main else ""),
        "value": round(args.batch / step_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": cfg,
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4), "measured_peak": round(hbm_meas / 1e9, 1),
                     "frac_measured": round(achieved / hbm_meas, 4)},
        "measured_peaks": {"hbm_read_GB_s": round(hbm_meas / 1e9, 1), "mfma_bf16_TFLOP_s": round(peaks["mfma_bf16_flop_per_s"] / 1e12, 1)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


def steady(args, shape_name: str, dtype: str, layers: int, context: int, decodes, prefills) -> dict:
    """Builds the shape with random weights in ``dtype`` ("bf16" or "fp32") and measures prefills (``tokens`` of one
    prompt in portions of ``portion``, through the step function) and steady decoding (``batch`` requests with prompts
    of ``prompt_len``, through the engine's loop): {"prefill": {key: {...}}, "decode": {key: (s per step, tokens held
    on average, bytes a step must read)}, "config": {...}}."""
    import torch
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_model, build_runner
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.sampling import SamplingParams
    from jllm_serve_amd.weights.random_init import random_source

    dev = torch.device("cuda:0")
    shape = shape_config(shape_name)
    full_layers = shape["num_hidden_layers"]
    if layers:
        shape["num_hidden_layers"] = layers
    cfg = parse_config(shape)
    run_dtype = "bfloat16" if dtype == "bf16" else "float32"
    t0 = time.time()
    source = random_source(shape, seed=0, gain_std=0.0, device=dev)
    model = build_model(cfg, source, run_dtype, dev, context)
    torch.cuda.synchronize()
    print(f"[bench] {dtype} model built in {time.time() - t0:.0f} s: {cfg.description}", file=sys.stderr, flush=True)
    work = Work(shape, dtype)
    chunk = 2048

    def held(p):  # positions a request of this point holds at most, in whole pages of 64
        head_start = p["batch"] * -(-p["prompt_len"] // chunk)  # tokens the first request decodes while the later ones still prefill
        return -(-(p["prompt_len"] + p["steps"] + p["warmup"] + 4 + head_start) // 64) * 64

    for p in decodes:
        if held(p) > context:
            raise SystemExit(f"bench.py: {p['key']}: {held(p)} positions per request do not fit the context of {context}")
    max_b = max([p["batch"] for p in decodes] + [1])
    pool = max([p["batch"] * held(p) for p in decodes] + [p["tokens"] + 64 for p in prefills])
    runner = build_runner(model, page_size=PAGE, pool_tokens=pool, max_requests=max_b, max_positions=context)
    V = work.V
    gen = torch.Generator().manual_seed(0)

    def prompt(n):
        return torch.randint(0, V, (n,), generator=gen).tolist()

    def sync():
        torch.cuda.synchronize()

    # ---- prefill: one prompt through the step function in portions, the logits of its last token
    prefill = {}
    for p in prefills:
        T, portion = p["tokens"], p["portion"]
        ptoks = prompt(T)
        cuts = list(range(0, T, portion))

        def once():
            for c in cuts:
                n = min(portion, T - c)
                runner.step([StepEntry("p", ptoks[c:c + n], [n - 1] if c + n == T else [])])
            runner.finish("p")

        for _ in range(2):
            once()
        sync()
        reps = 3
        t = time.perf_counter()
        for _ in range(reps):
            once()
        sync()
        s_ = (time.perf_counter() - t) / reps
        flops = work.flops(T, T * (T + 1) / 2, 1)
        prefill[p["key"]] = {"value": round(T / s_, 1), "tokens": T, "ms": round(s_ * 1e3, 3),
                             "frac": round(flops / s_ / FLOP_PEAK[dtype], 4), "flops": flops}
        print(f"[bench] {shape_name} {dtype} prefill {T} tokens in portions of {portion}: {s_ * 1e3:.1f} ms "
              f"({flops / s_ / 1e15:.3f} PFLOP/s)", file=sys.stderr, flush=True)

    # ---- decode: B requests with prompt_len-token prompts, through the engine loop
    def decode(p):
        B, k, w = p["batch"], p["steps"], p["warmup"]
        eng = Engine(runner, SchedulerConfig(max_batch_tokens=2 * chunk, prefill_chunk=chunk, max_running=B,
                                             max_positions=context))
        params = p.get("sampling") or SamplingParams.greedy_params(max_tokens=1, ignore_eos=True)
        params = params.with_max_tokens(k + w + 2 + B * -(-p["prompt_len"] // chunk))
        for _ in range(B):
            eng.add_request(prompt(p["prompt_len"]), params)
        while any(r.computed < len(r.prompt) for r in eng.requests.values()):
            eng.step()
        for _ in range(w):
            eng.step()
        sync()
        ctx0 = sum(r.computed for r in eng.requests.values())
        t = time.perf_counter()
        for _ in range(k):
            eng.step()
        sync()
        dt = time.perf_counter() - t
        ctx1 = sum(r.computed for r in eng.requests.values())
        assert len(eng.scheduler.running) == B and ctx1 - ctx0 == B * k, "every request decodes in every timed step"
        for r in list(eng.requests.values()):
            eng.cancel(r.rid)
        eng.step()
        return dt / k, (ctx0 + ctx1) / 2.0

    results = {}
    for p in decodes:
        step_s, held_mean = decode(p)
        by = work.decode_bytes(held_mean)
        results[p["key"]] = (step_s, held_mean, by)
        print(f"[bench] {shape_name} {dtype} decode {p['key']}: batch {p['batch']}, {held_mean / p['batch']:.0f} keys each: "
              f"{step_s * 1e3:.2f} ms/step = {p['batch'] / step_s:.1f} tok/s, {by / step_s / 1e12:.2f} TB/s",
              file=sys.stderr, flush=True)
    config = {"model": f"Qwen3-{shape_name.upper()} shape", "layers": work.L, "layers_in_shape": full_layers, "hidden": work.d,
              "heads": work.H, "kv_heads": work.Hkv, "head_dim": work.hd, "intermediate": work.F, "vocab": V,
              "batch": args.batch, "prompt_len": args.prompt_len, "context": context, "page_size": PAGE,
              "global_batch": args.batch, "seq_len": args.prompt_len, "parallelism": "single GPU"}
    del runner, model, source
    torch.cuda.empty_cache()
    return {"prefill": prefill, "decode": results, "config": config}


if __name__ == "__main__":
    sys.exit(main())
