"""The C++ host core (cache manager, scheduler) built with the address and undefined-behaviour
sanitizers and driven by random orders of requests (tests/host_core_check.cpp)."""
import os
import shutil
import subprocess

import pytest

from conftest import ROOT


def test_host_core_under_sanitizers(tmp_path):
    cxx = shutil.which("g++")
    if cxx is None:
        pytest.skip("no g++")
    host = os.path.join(ROOT, "denno-beta_amd", "csrc", "host")
    exe = str(tmp_path / "host_core_check")
    build = subprocess.run([cxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan",
                            "-I", host, os.path.join(ROOT, "tests", "host_core_check.cpp"),
                            os.path.join(host, "cache_manager.cpp"), os.path.join(host, "scheduler.cpp"), "-o", exe],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    # the sanitizer's runtime is linked statically, so that it need not be first among the
    # libraries the process loads
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0")
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "host core ok" in run.stdout
