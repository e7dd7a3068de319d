"""Traces for the replay tests: the same sequences cut in different ways, and the comparison
of what a replay wrote with the plain implementation."""
from __future__ import annotations

import random

import torch


def whole_trace(seqs):
    """Each request alone and whole, one step each."""
    return [{"step": i, "entries": [{"id": f"r{i}", "tokens": s, "want": list(range(len(s)))}], "end": [f"r{i}"]}
            for i, s in enumerate(seqs)]


def tail_decode_trace(seqs, tail=32):
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps = []
    for i, s in enumerate(seqs):
        head = max(1, len(s) - tail)
        steps.append({"step": len(steps), "entries": [{"id": f"r{i}", "tokens": s[:head], "want": list(range(head))}],
                      "end": []})
        for j in range(head, len(s)):
            steps.append({"step": len(steps), "entries": [{"id": f"r{i}", "tokens": s[j:j + 1], "want": [0]}],
                          "end": [f"r{i}"] if j == len(s) - 1 else []})
        if head == len(s):
            steps[-1]["end"] = [f"r{i}"]
    return steps


def chunk_trace(seqs, sizes=(2, 3, 5, 17, 2, 64, 7, 128, 2, 31)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for i, s in enumerate(seqs):
        pos, k = 0, i
        while pos < len(s):
            n = min(sizes[k % len(sizes)], len(s) - pos)
            k += 1
            steps.append({"step": len(steps),
                          "entries": [{"id": f"r{i}", "tokens": s[pos:pos + n], "want": list(range(n))}],
                          "end": [f"r{i}"] if pos + n == len(s) else []})
            pos += n
    return steps


def mixed_trace(seqs, seed, max_live=4, sizes=(1, 1, 1, 2, 3, 5, 17, 40)):
    """Up to `max_live` requests at a time: portions of some beside single tokens of others,
    requests left out of steps now and then, new ones starting as old ones end."""
    rng = random.Random(seed)
    pending, live, steps = list(range(len(seqs))), {}, []
    while pending or live:
        while pending and len(live) < max_live:
            live[pending.pop(0)] = 0
        entries, end = [], []
        for i in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue
            n = min(rng.choice(sizes), len(seqs[i]) - live[i])
            entries.append({"id": f"r{i}", "tokens": seqs[i][live[i]:live[i] + n], "want": list(range(n))})
            live[i] += n
            if live[i] == len(seqs[i]):
                end.append(f"r{i}")
                del live[i]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def max_live_tokens(steps, round_to=64):
    """The most tokens that live requests hold at any time, each rounded up to `round_to`."""
    held, worst = {}, 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // round_to) * round_to for n in held.values()))
        for name in st["end"]:
            held.pop(name, None)
    return worst


def replay(runner, steps):
    """Runs the steps in-process; -> {request id: [len, vocab] logits by position} (CPU)."""
    from denno_beta_amd.engine.replay import TraceReplayer
    rp = TraceReplayer(runner)
    rows, pos = {}, {}
    for st in steps:
        out = rp.run_step(st)
        out = out.cpu() if out is not None else None
        k = 0
        for e in st["entries"]:
            base = pos.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[base + w] = out[k]
                k += 1
            pos[e["id"]] = base + len(e["tokens"])
    return {rid: torch.stack([r[p] for p in sorted(r)]) for rid, r in rows.items()}


def collect_files(out_dir, steps, vocab):
    """The same from the <step>.f32 files that bin/trace_run wrote."""
    import numpy as np
    import os
    rows, pos = {}, {}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        out = None
        if wanted:
            a = np.fromfile(os.path.join(out_dir, f"{st['step']}.f32"), dtype="<f4")
            assert a.size == wanted * vocab, (st["step"], a.size, wanted, vocab)
            out = torch.from_numpy(a.reshape(wanted, vocab).copy())
        k = 0
        for e in st["entries"]:
            base = pos.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[base + w] = out[k]
                k += 1
            pos[e["id"]] = base + len(e["tokens"])
    return {rid: torch.stack([r[p] for p in sorted(r)]) for rid, r in rows.items()}


# Tolerances.  32-bit differs from the plain implementation by the order of its sums: absolute and relative
# bounds on logits of size about 1.  bfloat16 rounds every activation between kernels to 8 bits of mantissa, and
# what that does to a logit is measured against what a row's logits differ by among themselves (their standard
# deviation over the vocabulary, 0.14 to 0.8 with these random weights): over every bfloat16 comparison of these
# tests the worst logit was off by 0.030 of its row's spread and a comparison's mean by 0.0035.  A lost key, a
# wrong page or a neighbour's row move a logit by the spread itself.
TOL = {"float32": dict(atol=2e-5, rtol=1e-5)}
BF16_WORST, BF16_MEAN = 0.04, 0.007


def assert_close(got, want, dtype, what):
    got, want = got.float(), want.float()
    if dtype == "bfloat16":
        spread = want.std(dim=1, keepdim=True)
        diff = (got - want).abs() / spread
        worst, mean = diff.max().item(), diff.mean().item()
        if not (worst <= BF16_WORST and mean <= BF16_MEAN):
            at = (diff == diff.max()).nonzero()[0].tolist()
            raise AssertionError(f"{what}: bfloat16 logits differ by {worst:.4f} of a row's spread at worst (position {at[0]}, "
                                 f"token {at[1]}: got {got[at[0], at[1]].item()}, want {want[at[0], at[1]].item()}), "
                                 f"{mean:.5f} on average; the bounds are {BF16_WORST} and {BF16_MEAN}")
        return
    tol = TOL[dtype]
    diff = (got - want).abs()
    bound = tol["atol"] + tol["rtol"] * want.abs()
    if not bool((diff <= bound).all()):
        bad = (diff > bound).nonzero()
        first = bad[0].tolist()
        raise AssertionError(f"{what}: {len(bad)} logits differ; first at position {first[0]}, token {first[1]}: "
                             f"got {got[first[0], first[1]].item()}, want {want[first[0], first[1]].item()}; "
                             f"worst {diff.max().item():.3g}")
