"""bin/trace_run as a user runs it: a child process, steps on its standard input, logits in files."""
import json
import os
import subprocess
import sys

import pytest

import replay_util as U
from conftest import ROOT, TINY, seeded_tokens
from plain.gpt2_plain import PlainGPT2

pytestmark = pytest.mark.gpu


def run_trace(folder, dtype, out_dir, steps, *more):
    p = subprocess.Popen([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out",
                          str(out_dir), "--max-tokens", str(U.max_live_tokens(steps)), *more],
                         stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:      # the next step is sent only after `done <step>`
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        assert p.stdout.readline().strip() == f"done {st['step']}"
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    return U.collect_files(str(out_dir), steps, 1000)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run(model_folders, tmp_path, dtype):
    """Steps of single tokens come from captured HIP graphs, as in generation; with --no-graphs the same
    steps run kernel by kernel and must give the same bits."""
    import torch
    folder = model_folders("B", dtype)
    seqs = [seeded_tokens(40 + i, n, 1000) for i, n in enumerate((90, 33, 150, 64, 20))]
    steps = U.mixed_trace(seqs, seed=9)
    for st in U.tail_decode_trace(seqs[:2], 32):        # and two of them again, their last tokens one by one
        steps.append({"step": len(steps), "end": [x.replace("r", "t") for x in st["end"]],
                      "entries": [dict(e, id=e["id"].replace("r", "t")) for e in st["entries"]]})
    assert sum(all(len(e["tokens"]) == 1 for e in st["entries"]) for st in steps) > 40
    got = run_trace(folder, dtype, tmp_path / "out", steps)
    eager = run_trace(folder, dtype, tmp_path / "eager", steps, "--no-graphs")
    plain = PlainGPT2.from_folder(folder)
    for i, s in enumerate(seqs):
        U.assert_close(got[f"r{i}"], plain.logits(s), dtype, f"trace_run {dtype} request {i}")
        assert torch.equal(got[f"r{i}"], eager[f"r{i}"]), f"request {i}: graphs and kernel-by-kernel steps differ"
    for i in range(2):
        U.assert_close(got[f"t{i}"], plain.logits(seqs[i]), dtype, f"trace_run {dtype} request {i}, tail decoded")
        assert torch.equal(got[f"t{i}"], eager[f"t{i}"]), f"request {i}: graphs and kernel-by-kernel steps differ"
