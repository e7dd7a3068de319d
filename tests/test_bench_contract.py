"""bench.py's contract at the edges that need no GPU: more than one GPU is refused with one line and exit
code 2, and sampling options belong to the decode-only mode."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_one_line():
    p = _bench("--gpus", "2", "--steps", "3", "--warmup", "1")
    assert p.returncode == 2
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_sampling_options_go_with_the_decode_mode_only():
    p = _bench("--temperature", "0.8")
    assert p.returncode == 2 and "--only decode" in p.stdout
