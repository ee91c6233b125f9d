"""Decode and prefill throughput of the engine at the Qwen3-8B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch through the engine's own loop (scheduler, step function, paged
cache, kernels, device-side argmax). Prints one JSON line. Peaks used for the fractions are the published
MI355X figures: HBM 8 TB/s; dense MFMA 2.5 PFLOP/s for bf16, 157.3 TFLOP/s for fp32. Beside them the line gives the
same fractions against what this GPU delivered to two probes run at the start (a kernel that only streams memory
in, a kernel that only issues bf16 MFMAs): `frac_measured`. The default run also reports, under `points`, decoding
at batch 1 and 64 with their fractions, the float32 path of the same shape on fewer layers (`config` names both
counts), and the 14B and 32B request sets served to the end (`--no-serve` and `--no-fp32` leave them out).
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


SHAPES = {  # the Qwen3-8B / 14B / 32B layer sizes: (layers, hidden, heads, kv heads, head dim, intermediate, context)
    "8b": (36, 4096, 32, 8, 128, 12288, 8192),
    "14b": (40, 5120, 40, 8, 128, 17408, 8192),
    "32b": (64, 5120, 64, 8, 128, 25600, 16384),
}


def shape_config(name="8b"):
    """A config.json of the Qwen3-8B / 14B / 32B layer sizes."""
    L, d, H, Hkv, hd, F, ctx = SHAPES[name]
    return dict(model_type="qwen3", architectures=["Qwen3ForCausalLM"], num_hidden_layers=L, hidden_size=d,
                num_attention_heads=H, num_key_value_heads=Hkv, head_dim=hd, intermediate_size=F,
                vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False,
                max_position_embeddings=ctx)


def serve_workload(args) -> dict:
    """The 14B and 32B workloads: a set of requests served to the end by the engine (scheduler, mixed passes,
    paged cache near full). 14b: 32 requests, prompts uniform in 128..4096, 128 generated each. 32b: 64 prompts of
    1,024 tokens, 256 generated each, pool of exactly 64 x 1,280 positions."""
    import random

    import torch
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_model, build_runner
    from jllm_serve_amd.kernels import ops
    from jllm_serve_amd.sampling import SamplingParams
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
    runner = build_runner(model, page_size=16, pool_tokens=pool, max_requests=n_req, max_positions=ctx,
                          prefix_share=args.shared_prefix > 0)
    torch.cuda.synchronize()
    print(f"[bench] model built in {time.time() - t0:.0f} s: {cfg.description}", file=sys.stderr, flush=True)
    params = SamplingParams.greedy_params(max_tokens=gen, ignore_eos=True)

    def run():
        runner.cache.drop_cached()  # nothing of an earlier run is found again
        eng = Engine(runner, SchedulerConfig(max_batch_tokens=args.budget, prefill_chunk=args.budget, max_running=n_req, max_positions=ctx))
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
    out = {
        "metric": f"generated tok/s serving {n_req} requests to the end (Qwen3-{args.shape.upper()} shape, 1 GPU)",
        "value": round(generated / dt, 2), "unit": "tok/s", "n_gpus": 1, "steps": st["scheduler"]["passes"], "warmup": 1,
        "ms_per_step": round(dt * 1e3 / st["scheduler"]["passes"], 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": f"Qwen3-{args.shape.upper()} shape", "layers": cfg.num_layers, "layers_in_shape": SHAPES[args.shape][0],
                   "hidden": cfg.hidden, "heads": shape["num_attention_heads"], "kv_heads": shape["num_key_value_heads"],
                   "head_dim": shape["head_dim"], "intermediate": shape["intermediate_size"], "vocab": V,
                   "requests": n_req, "prompt_tokens": sum(lens), "generated_per_request": gen, "context": ctx,
                   "pool_tokens": pool, "page_size": 16, "pass_budget": args.budget, "shared_prefix": args.shared_prefix, "global_batch": n_req, "seq_len": max(lens), "parallelism": "single GPU"},
        "wall_s": round(dt, 3), "prompt_tok_per_s": round(sum(lens) / dt, 1), "preemptions": st["scheduler"]["preemptions"],
        "rows_per_pass": round(st["scheduler"]["rows_per_pass"], 1),
        "cached_prompt_tokens": int(sum(r.stats.get("cached_tokens", 0) for r in res)),
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
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--points", default="1,64", help="other decode batch sizes to report")
    ap.add_argument("--point-steps", type=int, default=24)
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="8b is the default run; 14b and 32b with --workload serve")
    ap.add_argument("--budget", type=int, default=8192, help="serve: rows per pass (prompt portions + decoding requests)")
    ap.add_argument("--shared-prefix", type=int, default=0,
                    help="serve: every prompt starts with the same N tokens and the cache shares their pages (0 = off)")
    ap.add_argument("--no-serve", action="store_true", help="steady: leave out the 14B and 32B request sets")
    ap.add_argument("--no-fp32", action="store_true", help="steady: leave out the float32 figures")
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
    points_b = sorted({int(p) for p in args.points.split(",") if p} | {args.batch})
    main_run = steady(args, args.dtype, args.layers, points_b, args.steps, args.warmup)
    step_s, mean_ctx, bytes_step = main_run["decode"][args.batch]
    achieved = bytes_step / step_s
    hbm_meas = peaks["hbm_read_bytes_per_s"]
    flop_meas = peaks["mfma_bf16_flop_per_s"] if args.dtype == "bf16" else None
    prefill = dict(main_run["prefill"])
    if flop_meas:
        prefill["frac_measured"] = round(prefill.pop("flops") / (prefill["ms"] * 1e-3) / flop_meas, 4)
    else:
        prefill.pop("flops")
    points = {}
    for B in points_b:
        if B == args.batch:
            continue
        s_, _, by = main_run["decode"][B]
        points[f"decode_b{B}"] = round(B / s_, 2)
        points[f"decode_b{B}_hbm_frac"] = round(by / s_ / HBM_PEAK, 4)
        points[f"decode_b{B}_hbm_frac_measured"] = round(by / s_ / hbm_meas, 4)
    cfg = dict(main_run["config"])
    if not args.no_fp32 and args.dtype == "bf16":
        f32 = steady(args, "fp32", args.fp32_layers, [args.batch], max(8, args.steps // 4), 2)
        fs, _, fby = f32["decode"][args.batch]
        points["fp32_prefill_tok_s"] = f32["prefill"]["value"]
        points["fp32_prefill_frac"] = f32["prefill"]["frac"]
        points[f"fp32_decode_b{args.batch}"] = round(args.batch / fs, 2)
        points[f"fp32_decode_b{args.batch}_hbm_frac"] = round(fby / fs / HBM_PEAK, 4)
        cfg["fp32_layers"] = f32["config"]["layers"]
    if not args.no_serve and args.dtype == "bf16" and not args.layers:
        for shape in ("14b", "32b"):
            sargs = argparse.Namespace(**{**vars(args), "shape": shape, "layers": 0, "shared_prefix": 0})
            r = serve_workload(sargs)
            points[f"serve_{shape}_tok_s"] = r["value"]
            points[f"serve_{shape}_prompt_tok_s"] = r["prompt_tok_per_s"]
            points[f"serve_{shape}_wall_s"] = r["wall_s"]
            points[f"serve_{shape}_preemptions"] = r["preemptions"]
            print(f"[bench] serve {shape}: {r['value']} generated tok/s, {r['wall_s']} s", file=sys.stderr, flush=True)
    out = {
        "metric": "decode tok/s at batch 8 (Qwen3-8B shape, 1 GPU)" if args.batch == 8 and args.shape == "8b" else f"decode tok/s at batch {args.batch}",
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


def steady(args, dtype: str, layers: int, points, steps: int, warmup: int) -> dict:
    """Builds the shape with random weights in ``dtype`` ("bf16" or "fp32") and measures a 2,048-token prefill and
    steady decoding at the batch sizes ``points``: {"prefill": {...}, "decode": {B: (s per step, mean context, bytes
    a step must read)}, "config": {...}}."""
    import torch
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_model, build_runner
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.sampling import SamplingParams
    from jllm_serve_amd.weights.random_init import random_source

    dev = torch.device("cuda:0")
    shape = shape_config(args.shape)
    full_layers = shape["num_hidden_layers"]
    if layers:
        shape["num_hidden_layers"] = layers
    cfg = parse_config(shape)
    run_dtype = "bfloat16" if dtype == "bf16" else "float32"
    t0 = time.time()
    source = random_source(shape, seed=0, gain_std=0.0, device=dev)
    page = 16
    max_b = max(points)
    model = build_model(cfg, source, run_dtype, dev, args.context)
    torch.cuda.synchronize()
    print(f"[bench] {dtype} model built in {time.time() - t0:.0f} s: {cfg.description}", file=sys.stderr, flush=True)
    passes_per_prompt = -(-args.prompt_len // 2048)
    head_start = max_b * passes_per_prompt  # tokens the first request decodes while the later ones still prefill
    total_steps = max(steps + warmup, args.point_steps + 4) + 2 + head_start
    per_req = -(-(args.prompt_len + total_steps) // 64) * 64
    pool = max(max_b * per_req, 2048 + 64)  # the 2,048-token prefill measured below has to fit as well
    runner = build_runner(model, page_size=page, pool_tokens=pool, max_requests=max_b, max_positions=args.context)
    L, d, H, Hkv, hd = cfg.num_layers, cfg.hidden, shape["num_attention_heads"], shape["num_key_value_heads"], shape["head_dim"]
    F, V = shape["intermediate_size"], shape["vocab_size"]
    esize = 2 if dtype == "bf16" else 4
    layer_params = (H * hd + 2 * Hkv * hd) * d + d * H * hd + 3 * d * F
    weight_bytes = (L * layer_params + V * d) * esize
    kv_bytes_per_token = 2 * L * Hkv * hd * esize
    gen = torch.Generator().manual_seed(0)

    def prompt(n):
        return torch.randint(0, V, (n,), generator=gen).tolist()

    def sync():
        torch.cuda.synchronize()

    # ---- prefill of 2,048 tokens: one step of the step function, logits of the last token
    T = 2048
    ptoks = prompt(T)
    for _ in range(2):
        runner.step([StepEntry("p", ptoks, [T - 1])])
        runner.finish("p")
    sync()
    reps = 3
    t = time.perf_counter()
    for _ in range(reps):
        runner.step([StepEntry("p", ptoks, [T - 1])])
        runner.finish("p")
    sync()
    prefill_s = (time.perf_counter() - t) / reps
    flops = 2.0 * T * L * layer_params + 2.0 * V * d + L * 4.0 * H * hd * (T * (T + 1) / 2)
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(flops / prefill_s / FLOP_PEAK[dtype], 4), "flops": flops}
    print(f"[bench] {dtype} prefill {T} tokens: {prefill_s * 1e3:.1f} ms", file=sys.stderr, flush=True)

    # ---- decode: B requests with prompt_len-token prompts, through the engine loop
    def decode(B, k, w):
        eng = Engine(runner, SchedulerConfig(max_batch_tokens=4096, prefill_chunk=2048, max_running=B,
                                             max_positions=args.context))
        params = SamplingParams.greedy_params(max_tokens=k + w + 2 + B * passes_per_prompt, ignore_eos=True)
        for _ in range(B):
            eng.add_request(prompt(args.prompt_len), params)
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
        mean_ctx = (ctx0 + ctx1) / 2.0
        return dt / k, mean_ctx

    results = {}
    for B in points:
        k, w = (steps, warmup) if B == args.batch else (args.point_steps, 4)
        step_s, mean_ctx = decode(B, k, w)
        results[B] = (step_s, mean_ctx, weight_bytes + kv_bytes_per_token * mean_ctx)
        print(f"[bench] {dtype} decode batch {B}: {step_s * 1e3:.2f} ms/step = {B / step_s:.1f} tok/s", file=sys.stderr, flush=True)
    config = {"model": f"Qwen3-{args.shape.upper()} shape", "layers": L, "layers_in_shape": full_layers, "hidden": d, "heads": H,
              "kv_heads": Hkv, "head_dim": hd, "intermediate": F, "vocab": V, "batch": args.batch,
              "prompt_len": args.prompt_len, "context": args.context, "page_size": page,
              "global_batch": args.batch, "seq_len": args.prompt_len, "parallelism": "single GPU"}
    del runner, model, source
    torch.cuda.empty_cache()
    return {"prefill": prefill, "decode": results, "config": config}


if __name__ == "__main__":
    sys.exit(main())
