#!/usr/bin/python3
"""Measurement: GPT-2 XL shape, random weights, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the engine (scheduler, step function, sampling): batch 8 from a
512-token context by default.  Every figure is the median of three blocks of K steps (of three runs for
the prefill).  One JSON line: decoded tokens a second, the prefill of 2,048 tokens (two prompts of 1,024
in one step), the decode step's share of the HBM roofline, decoding at batch 1 and 64 (`points`: tokens a
second; `point_details`: milliseconds, bytes and share of the roofline of each), and the 32-bit engine's
decode steps and prefill (`fp32`).  Peaks are the published ones of MI355X.

    python bench.py --only decode|prefill [--kernel-times]   one workload; with --kernel-times kernel by
                                                             kernel, each launch between two HIP events
    python bench.py --only serving [--dtype float32]         BASELINE.json's configs[3] through the scheduler
    python bench.py --only replay [--sequences 8] [--shape xl]   BASELINE.json's configs[4] (or configs[2]'s sizes)
                                                             against the plain implementation, in four ways of cutting
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
SHORT = {"bfloat16": "bf16", "float32": "fp32"}


def baseline_config(index, n_layer=0):
    """The sizes that BASELINE.json's configs[index] names in words -> (config.json keys, its layers)."""
    import re
    with open(os.path.join(ROOT, "BASELINE.json")) as f:
        text = json.load(f)["configs"][index]
    num = lambda key: int(re.search(key + r"=(\d+)", text).group(1))   # noqa: E731
    cfg = dict(architectures=["GPT2LMHeadModel"], n_layer=num("n_layer"), n_embd=num("n_embd"), n_head=num("n_head"),
               n_inner=num("n_inner"), vocab_size=num("vocab_size"), n_positions=num("n_positions"),
               layer_norm_epsilon=1e-5, activation_function="gelu_new")
    full = cfg["n_layer"]
    if n_layer:
        cfg["n_layer"] = n_layer
    return cfg, full


class Workloads:
    """The decode and prefill measurements on one runner."""

    def __init__(self, a, dtype):
        import torch
        from denno_beta_amd.config import EngineOptions
        from denno_beta_amd.engine import ModelRunner
        self.torch, self.a, self.dtype = torch, a, dtype
        self.cfg, self.full_layers = baseline_config({"xl": 2, "large": 3, "medium": 4}[a.shape], a.layers)
        P = self.cfg["n_positions"]
        live = max(64, a.batch)
        self.opts = EngineOptions(dtype=dtype, page_size=a.page_size, cache_tokens=live * P, max_live=live, max_batch_tokens=4096,
                                  prefill_chunk=1024, use_graphs=not (a.no_graphs or a.kernel_times), seed=0,
                                  norms_inside_products=not a.norm_kernels, deferred_sums=not a.no_deferred_sums)
        self.runner = ModelRunner.from_random(self.cfg, seed=0, options=self.opts, stored=dtype)
        self.gen = torch.Generator().manual_seed(0)

    def prompt(self, n):
        return self.torch.randint(0, self.cfg["vocab_size"], (n,), generator=self.gen).tolist()

    def decode(self, batch, steps, warmup, blocks=3):
        """-> {ms, tok_s, bytes, frac, mean_context}: the median block of `steps` steps."""
        from denno_beta_amd.engine import Engine, SamplingParams
        a, P, sync = self.a, self.cfg["n_positions"], self.torch.cuda.synchronize
        steps = max(1, min(steps, (P - a.context - warmup - 2) // blocks))
        eng = Engine(self.runner, self.opts)
        # greedy, unless --only decode names other sampling options (what the sampling kernels cost a step)
        sp = SamplingParams(max_tokens=P, temperature=getattr(a, "temperature", 0.0), top_k=getattr(a, "top_k", None),
                            top_p=getattr(a, "top_p", None), repetition_penalty=getattr(a, "repetition_penalty", None),
                            seed=3, ignore_eos=True)
        rids = [eng.add_request(self.prompt(a.context), sp) for _ in range(batch)]
        while any(eng.scheduler.computed(r) < a.context for r in rids):
            eng.step()
        for _ in range(warmup):
            eng.step()
        times = []
        for _ in range(blocks):
            sync()
            t0 = time.perf_counter()
            for _ in range(steps):
                eng.step()
            sync()
            times.append((time.perf_counter() - t0) / steps)
        assert all(len(eng.requests[r].generated) >= blocks * steps for r in rids)
        for r in rids:
            eng.abort(r)
        order = sorted(range(blocks), key=lambda i: times[i])
        mid = order[blocks // 2]
        mean_ctx = a.context + 1 + warmup + mid * steps + (steps - 1) / 2.0
        nbytes = self.runner.model.weight_bytes() + batch * mean_ctx * self.runner.cache.bytes_per_token()
        t = times[mid]
        return {"ms": t * 1e3, "tok_s": batch / t, "bytes": nbytes, "frac": nbytes / t / 1e9 / HBM_PEAK_GBS,
                "mean_context": mean_ctx, "steps": steps}

    def prefill(self, reps=3, prompts=2):
        """-> {value, tokens, ms, frac}: `prompts` prompts of 1,024 tokens in one step (two: the 2,048 tokens
        of the contract), the median of `reps`."""
        from denno_beta_amd.engine import StepEntry
        runner, sync = self.runner, self.torch.cuda.synchronize
        times = []
        for i in range(reps + 1):
            seqs = [self.prompt(1024) for _ in range(prompts)]
            for j in range(prompts):
                runner.start_request(1000 + j)
            sync()
            t0 = time.perf_counter()
            runner.step([StepEntry(1000 + j, seqs[j], [1023]) for j in range(prompts)])
            sync()
            times.append(time.perf_counter() - t0)
            for j in range(prompts):
                runner.end_request(1000 + j)
        t = statistics.median(times[1:])
        cfg = self.cfg
        V, E = cfg["vocab_size"], cfg["n_embd"]
        mat = sum(w.numel() for w in _layer_matrices(runner))
        tokens = 1024 * prompts
        flops = 2.0 * tokens * mat + 2.0 * prompts * V * E + cfg["n_layer"] * prompts * (4.0 * E * 1024 * 1025 / 2)
        return {"value": tokens / t, "tokens": tokens, "ms": t * 1e3, "frac": flops / t / MFMA_PEAK[SHORT[self.dtype]]}


def _layer_matrices(runner):
    from denno_beta_amd.parts import Linear
    seen = []
    for b in runner.model.blocks:
        for p in b.parts():
            for v in vars(p).values():
                if isinstance(v, Linear):
                    seen.append(v.weight)
    return seen


def kernel_table(what):
    """Prints the per-kernel shares that ops.time_launches measured."""
    from denno_beta_amd.kernels import ops
    times = ops.launch_times()
    total = sum(ms for _, ms in times.values())
    print(f"{what}: {total:.3f} ms in {sum(n for n, _ in times.values())} launches (each between two events)")
    for name, (n, ms) in sorted(times.items(), key=lambda kv: -kv[1][1]):
        print(f"  {ms / total * 100:5.1f} %  {ms / n * 1e3:8.1f} us x {n:5d}  {name}")


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
    ap.add_argument("--no-deferred-sums", action="store_true",
                    help="every product into the stream adds its own sum (steps of 65 to 256 rows; for comparison)")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64, the prefill and the 32-bit engine")
    ap.add_argument("--kernel-times", action="store_true",
                    help="with --only decode or prefill: every launch between two HIP events (no graphs), and a "
                         "table of each kernel's share")
    ap.add_argument("--sequences", type=int, default=8, help="--only replay: how many of the eight sequences")
    ap.add_argument("--page-size", type=int, default=16, help="tokens in a page of the cache (decode and prefill)")
    ap.add_argument("--prompts", type=int, default=2, help="--only prefill: prompts of 1,024 tokens in the one step")
    ap.add_argument("--temperature", type=float, default=0.0, help="--only decode: sampling instead of greedy (0: greedy)")
    ap.add_argument("--top-k", type=int, default=None, help="--only decode, with --temperature")
    ap.add_argument("--top-p", type=float, default=None, help="--only decode, with --temperature")
    ap.add_argument("--repetition-penalty", type=float, default=None, help="--only decode: penalties over each request's tokens")
    ap.add_argument("--shape", choices=["xl", "large", "medium"], default=None,
                    help="--only decode / prefill / replay: the layer sizes of BASELINE.json's configs[2], [3] or [4] "
                         "(default xl; for replay medium)")
    ap.add_argument("--only", choices=["decode", "prefill", "serving", "replay"], default=None,
                    help="run one workload and print a short line (decode, prefill: for profiling; serving: "
                         "BASELINE.json's configs[3], GPT-2 Large shape, 64 requests through the scheduler; replay: "
                         "configs[4], GPT-2 Medium shape, against the plain implementation)")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        sys.exit(2)
    if a.only == "serving":
        return serving(a)
    if a.only == "replay":
        a.shape = a.shape or "medium"      # (configs[4] as written; --shape xl: the same replay at configs[2]'s sizes)
        return replay(a)
    a.shape = a.shape or "xl"

    if a.only != "decode" and (a.temperature or a.top_k or a.top_p or a.repetition_penalty):
        print("bench.py: sampling options go with --only decode (the contract's line is greedy)")
        sys.exit(2)
    w = Workloads(a, a.dtype)
    if a.only in ("prefill", "decode"):
        from denno_beta_amd.kernels import ops
        if a.only == "prefill":
            w.prefill(1, a.prompts)
            if a.kernel_times:
                ops.time_launches(True)
            r = w.prefill(1 if a.kernel_times else 3, a.prompts)
            print(json.dumps({"prefill_ms": r["ms"], "tokens": r["tokens"], "tok_s": r["value"], "frac": r["frac"]}))
        else:
            if a.kernel_times:
                w.decode(a.batch, 2, 2, blocks=1)
                ops.time_launches(True)
            r = w.decode(a.batch, a.steps, a.warmup, blocks=1 if a.kernel_times else 3)
            print(json.dumps({"decode_ms_per_step": r["ms"], "batch": a.batch, "mean_context": r["mean_context"],
                              "frac": r["frac"]}))
        if a.kernel_times:
            kernel_table(f"{a.only}, {a.dtype}")
        return

    main_point = w.decode(a.batch, a.steps, a.warmup)
    cfg, short = w.cfg, SHORT[a.dtype]
    out = {
        "metric": "GPT-2 XL decode tokens/s (batch 8, context 512)", "value": main_point["tok_s"], "unit": "tokens/s",
        "n_gpus": 1, "steps": main_point["steps"], "warmup": a.warmup, "ms_per_step": main_point["ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": short, "data": "synthetic",
        "config": {"model": f"gpt2-{a.shape}-shape", "n_layer": cfg["n_layer"], "n_layer_full": w.full_layers,
                   "n_embd": cfg["n_embd"], "n_head": cfg["n_head"], "n_inner": cfg["n_inner"],
                   "vocab_size": cfg["vocab_size"], "n_positions": cfg["n_positions"], "global_batch": a.batch,
                   "seq_len": a.context, "page_size": w.opts.page_size, "weights": "random N(0,0.02)",
                   "graphs": w.opts.use_graphs, "timing": "median of 3 blocks", "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": main_point["bytes"] / main_point["ms"] / 1e6, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": main_point["frac"]},
    }
    if not a.no_points:
        out["prefill"] = w.prefill()
        b1 = w.decode(1, min(a.steps, 100), a.warmup)
        b64 = w.decode(64, min(a.steps, 50), a.warmup)
        out["points"] = {"decode_b1": b1["tok_s"], "decode_b64": b64["tok_s"]}
        keep = lambda r: {k: r[k] for k in ("ms", "tok_s", "bytes", "frac")}   # noqa: E731
        out["point_details"] = {"decode_b1": keep(b1), f"decode_b{a.batch}": keep(main_point), "decode_b64": keep(b64)}
        if a.dtype == "bfloat16":
            # the true 32-bit engine at the same sizes: every product in the plain kernels
            del w
            import torch
            torch.cuda.empty_cache()
            f = Workloads(a, "float32")
            f1, f8 = f.decode(1, min(a.steps, 10), 2), f.decode(8, min(a.steps, 10), 2)
            out["fp32"] = {"decode_b1": keep(f1), "decode_b8": keep(f8), "prefill": f.prefill()}
    print(json.dumps(out))


def large_config():
    return baseline_config(3)[0]


def serving(a):
    """GPT-2 Large shape, random weights: 64 requests with prompt lengths uniform in [16, 768], 256
    generated tokens each, greedy, continuous batching with prompt portions of 512.  After the timed
    run four of the requests run again, each alone: their tokens must be the same (32-bit: exactly; in
    bfloat16 a step's kernels depend on its rows, so the count of equal tokens is reported, and the served
    tokens are checked against the 32-bit engine wherever its lead is clear of bfloat16's rounding)."""
    import torch
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import Engine, SamplingParams
    cfg = large_config()
    opts = EngineOptions(dtype=a.dtype, page_size=16, cache_tokens=64 * 1024, max_live=64, max_batch_tokens=2048,
                         prefill_chunk=512, use_graphs=not a.no_graphs, seed=0, norms_inside_products=not a.norm_kernels, deferred_sums=not a.no_deferred_sums)
    eng = Engine.from_random(cfg, 0, opts, stored=a.dtype)
    gen = torch.Generator().manual_seed(1)
    lengths = torch.randint(16, 769, (64,), generator=gen).tolist()
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=gen).tolist() for n in lengths]
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
    records = list(eng.records)
    same = []
    for i in (0, 21, 42, 63):
        alone = eng.generate([prompts[i]], sp)[0]
        first_other = next((j for j in range(256) if alone[j] != out[i][j]), 256)
        same.append(first_other)
    if a.dtype == "float32" and min(same) < 256:
        raise SystemExit(f"serving: a request's tokens differ from its run alone (equal tokens before the first "
                         f"difference, of 256: {same})")
    clear_share = None
    if a.dtype == "bfloat16":
        # What can be asked of bfloat16: the 32-bit engine on the same weights, fed each request's prompt and the
        # tokens that were served, says at every generated position which token leads and by how much; where the
        # lead is clear of bfloat16's rounding (twice 0.04 of the row's spread, the bound of the replay tests) the
        # served token must be that one.
        from denno_beta_amd.engine import ModelRunner, StepEntry
        del eng
        r32 = ModelRunner.from_random(cfg, 0, EngineOptions(dtype="float32", page_size=16, cache_tokens=1024, max_live=1,
                                                            use_graphs=False), stored="bfloat16")
        clear = wrong = 0
        for rid, i in enumerate((0, 21, 42, 63)):
            seq = prompts[i] + out[i][:-1]
            r32.start_request(rid)
            logits = r32.step([StepEntry(rid, seq, list(range(len(prompts[i]) - 1, len(seq))))])
            r32.end_request(rid)
            top = logits.topk(2, dim=1)
            sure = (top.values[:, 0] - top.values[:, 1]) > 2 * 0.04 * logits.std(dim=1)
            served = torch.tensor(out[i], device=logits.device)
            clear += int(sure.sum())
            wrong += int((served != top.indices[:, 0])[sure].sum())
        clear_share = clear / (4 * 256)
        if wrong:
            raise SystemExit(f"serving: {wrong} served tokens differ from the 32-bit engine's where its lead is clear "
                             f"({clear} such positions of {4 * 256})")
    print(json.dumps({
        "workload": "GPT-2 Large shape, 64 requests, prompts U[16,768], 256 new tokens, prefill portions of 512",
        "seconds": dt, "generated_tokens": 64 * 256, "generated_tokens_per_s": 64 * 256 / dt,
        "prompt_tokens": sum(lengths), "all_tokens_per_s": (64 * 256 + sum(lengths)) / dt, "steps": steps,
        "mean_rows_per_step": sum(r.rows for r in records) / steps,
        "mixed_steps": sum(1 for r in records if r.decode_rows and r.prefill_rows),
        "preemptions": sum(r.preempted for r in records), "dtype": a.dtype,
        "tokens_equal_to_the_run_alone_before_the_first_difference": same,
        "share_of_positions_where_the_32_bit_lead_is_clear_all_served_as_it_says": clear_share}))


def replay(a):
    """BASELINE.json's configs[4] (GPT-2 Medium shape; --shape xl: configs[2]'s sizes, all 48 layers): random
    weights stored in 32-bit, seeded sequences of 1,024 tokens replayed whole, token by token, in portions of 128 and mixed (four live requests, pages
    used again), every logit compared with the plain implementation's; and the cuttings with each other."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import replay_util as U
    from plain.gpt2_plain import PlainGPT2
    from denno_beta_amd.config import EngineOptions
    from denno_beta_amd.engine import ModelRunner
    from denno_beta_amd.engine.replay import TraceReplayer
    from denno_beta_amd.weights import write_model_folder
    import tempfile
    cfg, full = baseline_config({"xl": 2, "large": 3, "medium": 4}[a.shape], a.layers)
    V, n = cfg["vocab_size"], cfg["n_positions"]
    seqs = [torch.randint(0, V, (n,), generator=torch.Generator().manual_seed(100 + i)).tolist()
            for i in range(a.sequences)]
    token_by_token = []
    for base in range(0, len(seqs), 4):          # four requests live at a time, a token of each per step
        group = list(range(base, min(base + 4, len(seqs))))
        for t in range(n):
            token_by_token.append({"step": len(token_by_token), "end": [f"r{i}" for i in group] if t == n - 1 else [],
                                   "entries": [{"id": f"r{i}", "tokens": seqs[i][t:t + 1], "want": [0]} for i in group]})
    traces = {"whole": U.whole_trace(seqs), "token by token": token_by_token,
              "portions of 128": U.chunk_trace(seqs, sizes=(128,)),
              "mixed": U.mixed_trace(seqs, seed=3, sizes=(1, 1, 1, 2, 5, 17, 40, 128))}
    result = {"workload": f"GPT-2 {a.shape} shape, {cfg['n_layer']} of {full} layers, {len(seqs)} sequences of {n} tokens"}
    with tempfile.TemporaryDirectory() as folder:
        print("replay: writing the model and running the plain implementation ...", file=sys.stderr, flush=True)
        write_model_folder(folder, cfg, 4, "float32")
        plain = PlainGPT2.from_folder(folder)
        want = []
        for i, s in enumerate(seqs):
            want.append(plain.logits(s, by_head=True).cuda())
            print(f"replay: plain logits of sequence {i}", file=sys.stderr, flush=True)
        for dtype in ("float32", "bfloat16"):
            whole = None
            for kind, steps in traces.items():
                tokens = U.max_live_tokens(steps)
                runner = ModelRunner.from_folder(folder, EngineOptions(dtype=dtype, page_size=16, cache_tokens=tokens,
                                                                       max_live=4), cast_matrices=True)
                rp = TraceReplayer(runner)
                got = [torch.empty_like(wt) for wt in want]
                pos = {}
                for st in steps:
                    out = rp.run_step(st)
                    k = 0
                    for e in st["entries"]:
                        i, base = int(e["id"][1:]), pos.get(e["id"], 0)
                        m = len(e["want"])
                        got[i][torch.tensor([base + x for x in e["want"]], device="cuda")] = out[k:k + m]
                        k += m
                        pos[e["id"]] = base + len(e["tokens"])
                runner.cache.manager.check()
                worst = max((g - wt).abs().max().item() for g, wt in zip(got, want))
                # the same against what a row's logits differ by among themselves (their standard deviation)
                rel = [(g - wt).abs() / wt.std(dim=1, keepdim=True) for g, wt in zip(got, want)]
                agree = sum((g.argmax(1) == wt.argmax(1)).sum().item() for g, wt in zip(got, want)) / (len(seqs) * n)
                entry = {"worst_difference_from_plain": worst, "greedy_token_agreement": agree,
                         "worst_of_a_rows_spread": max(r.max().item() for r in rel),
                         "mean_of_a_rows_spread": sum(r.mean().item() for r in rel) / len(rel),
                         "steps": len(steps), "pages_used_again": runner.cache.manager.reuse_count(0)}
                if whole is None:
                    whole = got
                else:
                    entry["equal_to_whole_bit_for_bit"] = all(torch.equal(g, wg) for g, wg in zip(got, whole))
                    entry["worst_difference_from_whole"] = max((g - wg).abs().max().item() for g, wg in zip(got, whole))
                result[f"{dtype}, {kind}"] = entry
                print(f"replay: {dtype}, {kind}: {entry}", file=sys.stderr, flush=True)
                del runner, rp
                if kind != "whole":
                    del got
            del whole
    result["largest_logit"] = max(wt.abs().max().item() for wt in want)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
