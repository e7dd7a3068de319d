#!/usr/bin/python3
"""Measurement: GPT-2 XL shape, random weights, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the engine (scheduler, step function, sampling): batch 8 from a
512-token context by default.  One JSON line: decoded tokens a second, the prefill of 2,048
tokens (two prompts of 1,024 in one step), the decode step's share of the HBM roofline, and
decoding at batch 1 and 64.  Peaks are the published ones of MI355X.
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}


def xl_config(n_layer):
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "BASELINE.json")) as f:
        text = json.load(f)["configs"][2]
    # the sizes that BASELINE.json's configs[2] names in words
    import re
    num = lambda key: int(re.search(key + r"=(\d+)", text).group(1))   # noqa: E731
    cfg = dict(architectures=["GPT2LMHeadModel"], n_layer=num("n_layer"), n_embd=num("n_embd"), n_head=num("n_head"),
               n_inner=num("n_inner"), vocab_size=num("vocab_size"), n_positions=num("n_positions"),
               layer_norm_epsilon=1e-5, activation_function="gelu_new")
    full = cfg["n_layer"]
    if n_layer:
        cfg["n_layer"] = n_layer
    return cfg, full


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=512)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0: all)")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--norm-kernels", action="store_true",
                    help="run every norm as a kernel of its own, also in steps of few rows (for comparisons)")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    ap.add_argument("--only", choices=["decode", "prefill", "serving"], default=None,
                    help="run one workload and print a short line (decode, prefill: for profiling; serving: "
                         "BASELINE.json's configs[3], GPT-2 Large shape, 64 requests through the scheduler)")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        sys.exit(2)

    import torch
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import Engine, ModelRunner, SamplingParams, StepEntry

    if a.only == "serving":
        return serving(a)
    cfg, full_layers = xl_config(a.layers)
    V, E, P = cfg["vocab_size"], cfg["n_embd"], cfg["n_positions"]
    if a.context + a.warmup + a.steps + 1 > P:
        a.steps = P - a.context - a.warmup - 1
    live = max(64, a.batch)
    opts = EngineOptions(dtype=a.dtype, page_size=16, cache_tokens=live * P, max_live=live, max_batch_tokens=4096,
                         prefill_chunk=1024, use_graphs=not a.no_graphs, seed=0, norms_inside_products=not a.norm_kernels)
    runner = ModelRunner.from_random(cfg, seed=0, options=opts, stored=a.dtype)
    gen = torch.Generator().manual_seed(0)
    prompt = lambda n: torch.randint(0, V, (n,), generator=gen).tolist()   # noqa: E731
    sync = torch.cuda.synchronize

    def decode_point(batch, steps, warmup):
        eng = Engine(runner, opts)
        sp = SamplingParams(max_tokens=P, temperature=0.0, ignore_eos=True)
        rids = [eng.add_request(prompt(a.context), sp) for _ in range(batch)]
        while any(eng.scheduler.computed(r) < a.context for r in rids):
            eng.step()
        for _ in range(warmup):
            eng.step()
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            eng.step()
        sync()
        dt = time.perf_counter() - t0
        assert all(len(eng.requests[r].generated) >= steps for r in rids)
        mean_ctx = a.context + 1 + warmup + (steps - 1) / 2.0
        for r in rids:
            eng.abort(r)
        return dt / steps, mean_ctx

    def prefill_point(reps=3):
        times = []
        for i in range(reps + 1):
            seqs = [prompt(1024), prompt(1024)]
            for j in range(2):
                runner.start_request(1000 + j)
            sync()
            t0 = time.perf_counter()
            runner.step([StepEntry(1000 + j, seqs[j], [1023]) for j in range(2)])
            sync()
            times.append(time.perf_counter() - t0)
            for j in range(2):
                runner.end_request(1000 + j)
        return sorted(times[1:])[len(times[1:]) // 2]

    if a.only == "prefill":
        t = prefill_point()
        print(json.dumps({"prefill_ms": t * 1e3, "tokens": 2048}))
        return
    step_s, mean_ctx = decode_point(a.batch, a.steps, a.warmup)
    if a.only == "decode":
        print(json.dumps({"decode_ms_per_step": step_s * 1e3, "batch": a.batch, "mean_context": mean_ctx}))
        return
    weight_bytes = runner.model.weight_bytes()
    kv_bytes = a.batch * mean_ctx * runner.cache.bytes_per_token()
    achieved = (weight_bytes + kv_bytes) / step_s / 1e9
    short = "bf16" if a.dtype == "bfloat16" else "fp32"
    out = {
        "metric": "GPT-2 XL decode tokens/s (batch 8, context 512)", "value": a.batch / step_s, "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": step_s * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": short, "data": "synthetic",
        "config": {"model": "gpt2-xl-shape", "n_layer": cfg["n_layer"], "n_layer_full": full_layers, "n_embd": E,
                   "n_head": cfg["n_head"], "n_inner": cfg["n_inner"], "vocab_size": V, "n_positions": P,
                   "global_batch": a.batch, "seq_len": a.context, "page_size": opts.page_size,
                   "weights": "random N(0,0.02)", "graphs": opts.use_graphs, "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS},
    }
    if not a.no_points:
        t = prefill_point()
        mat = sum(w.numel() for w in _layer_matrices(runner))
        flops = 2.0 * 2048 * mat + 2.0 * 2 * V * E + cfg["n_layer"] * 2 * (4.0 * E * 1024 * 1025 / 2)
        out["prefill"] = {"value": 2048 / t, "tokens": 2048, "ms": t * 1e3, "frac": flops / t / MFMA_PEAK[short]}
        b1, _ = decode_point(1, min(a.steps, 100), a.warmup)
        b64, _ = decode_point(64, min(a.steps, 50), a.warmup)
        out["points"] = {"decode_b1": 1 / b1, "decode_b64": 64 / b64}
    print(json.dumps(out))


def serving(a):
    """GPT-2 Large shape, random weights: 64 requests with prompt lengths uniform in [16, 768], 256
    generated tokens each, greedy, continuous batching with prompt portions of 512."""
    import torch
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import Engine, SamplingParams
    cfg = dict(architectures=["GPT2LMHeadModel"], n_layer=36, n_embd=1280, n_head=20, n_inner=5120, vocab_size=50257,
               n_positions=1024, layer_norm_epsilon=1e-5, activation_function="gelu_new")
    opts = EngineOptions(dtype=a.dtype, page_size=16, cache_tokens=64 * 1024, max_live=64, max_batch_tokens=2048,
                         prefill_chunk=512, use_graphs=not a.no_graphs, seed=0, norms_inside_products=not a.norm_kernels)
    eng = Engine.from_random(cfg, 0, opts, stored=a.dtype)
    gen = torch.Generator().manual_seed(1)
    lengths = torch.randint(16, 769, (64,), generator=gen).tolist()
    prompts = [torch.randint(0, 50257, (n,), generator=gen).tolist() for n in lengths]
    sp = SamplingParams(max_tokens=256, temperature=0.0, ignore_eos=True)
    eng.generate(prompts[:2], SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True))   # warm-up
    eng.records.clear()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = eng.generate(prompts, sp)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert all(len(o) == 256 for o in out)
    steps = len(eng.records)
    print(json.dumps({
        "workload": "GPT-2 Large shape, 64 requests, prompts U[16,768], 256 new tokens, prefill portions of 512",
        "seconds": dt, "generated_tokens": 64 * 256, "generated_tokens_per_s": 64 * 256 / dt,
        "prompt_tokens": sum(lengths), "all_tokens_per_s": (64 * 256 + sum(lengths)) / dt, "steps": steps,
        "mean_rows_per_step": sum(r.rows for r in eng.records) / steps,
        "mixed_steps": sum(1 for r in eng.records if r.decode_rows and r.prefill_rows),
        "preemptions": sum(r.preempted for r in eng.records), "dtype": a.dtype}))


def _layer_matrices(runner):
    from denno_beta_amd.parts import Linear
    seen = []
    for b in runner.model.blocks:
        for p in b.parts():
            for v in vars(p).values():
                if isinstance(v, Linear):
                    seen.append(v.weight)
    return seen


if __name__ == "__main__":
    main()
