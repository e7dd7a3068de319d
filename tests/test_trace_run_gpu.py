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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run(model_folders, tmp_path, dtype):
    folder = model_folders("B", dtype)
    seqs = [seeded_tokens(40 + i, n, 1000) for i, n in enumerate((90, 33, 150, 64, 20))]
    steps = U.mixed_trace(seqs, seed=9)
    out_dir = tmp_path / "out"
    p = subprocess.Popen([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out",
                          str(out_dir), "--max-tokens", str(U.max_live_tokens(steps))],
                         stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for st in steps:      # the next step is sent only after `done <step>`
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        assert p.stdout.readline().strip() == f"done {st['step']}"
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    got = U.collect_files(str(out_dir), steps, 1000)
    plain = PlainGPT2.from_folder(folder)
    for i, s in enumerate(seqs):
        U.assert_close(got[f"r{i}"], plain.logits(s), dtype, f"trace_run {dtype} request {i}")
