"""Compiling and loading the native libraries.

Two kinds: the host core (C++, g++) and the kernel libraries (HIP for gfx950, hipcc), one
shared object per kernel source file, so a program compiles only what it uses.  A library is
compiled at its first use if no built file matches its sources (the file name carries a hash
of sources and flags), into `_lib/` inside the package, or into a per-user folder under the
temporary directory when the package is read-only.  Nothing here falls back to another
implementation: a library that cannot be built or loaded raises.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

_PKG = os.path.dirname(os.path.realpath(__file__))
_CSRC = os.path.join(_PKG, "csrc")

HIP_ARCH = "gfx950"
HIP_FLAGS = ["--offload-arch=" + HIP_ARCH, "-O3", "-std=c++17", "-shared", "-fPIC",
             # hipcc -O3 must not form packed 32-bit float instructions on this target
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             # a kernel's first arguments arrive in scalar registers with the launch, where it would otherwise
             # begin by loading them: a trip to memory less in front of every kernel of a decode step
             "-mllvm", "-amdgpu-kernarg-preload-count=16",
             # the compiler's account of every kernel's registers, from which `spilling_kernels` reads
             "-Rpass-analysis=kernel-resource-usage"]
HOST_FLAGS = ["-std=c++17", "-O2", "-shared", "-fPIC", "-Wall", "-Wextra"]

# name -> (compiler kind, sources relative to csrc/, headers that the hash covers too)
LIBRARIES = {
    "host": ("host", ["host/cache_manager.cpp", "host/scheduler.cpp", "host/c_api.cpp"],
             ["host/cache_manager.h", "host/scheduler.h"]),
    "elementwise": ("hip", ["kernels/elementwise.hip"], ["kernels/common.h"]),
    "gemm": ("hip", ["kernels/gemm.hip", "kernels/gemm_plain.hip", "kernels/gemm_skinny.hip", "kernels/gemm_tiled.hip",
                     "kernels/gemm_direct.hip"], ["kernels/common.h", "kernels/gemm_common.h"]),
    "attention": ("hip", ["kernels/attention.hip"], ["kernels/common.h", "kernels/attention.h"]),
    "sampling": ("hip", ["kernels/sampling.hip"], ["kernels/common.h"]),
}

_loaded = {}
_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def _say(msg):
    print(f"[denno-beta_amd] {msg}", file=sys.stderr, flush=True)


_lib_dir_cached = None
_dir_lock = threading.Lock()


def _lib_dir():
    global _lib_dir_cached
    with _dir_lock:
        if _lib_dir_cached is None:
            d = os.path.join(_PKG, "_lib")
            try:
                os.makedirs(d, exist_ok=True)
                fd, probe = tempfile.mkstemp(dir=d)
                os.close(fd)
                os.remove(probe)
            except OSError:
                d = os.path.join(tempfile.gettempdir(), f"denno-beta_amd-{os.getuid()}", "_lib")
                os.makedirs(d, exist_ok=True)
            _lib_dir_cached = d
        return _lib_dir_cached


def _digest(name):
    kind, sources, headers = LIBRARIES[name]
    h = hashlib.sha256()
    h.update(" ".join(HIP_FLAGS if kind == "hip" else HOST_FLAGS).encode())
    for rel in list(sources) + list(headers):
        with open(os.path.join(_CSRC, rel), "rb") as f:
            h.update(rel.encode() + b"\0" + f.read())
    return h.hexdigest()[:12]


def _find_built(name):
    """The built file that matches the present sources, in the package or the fallback folder."""
    fname = f"libdenno_{name}-{_digest(name)}.so"
    for d in (os.path.join(_PKG, "_lib"),
              os.path.join(tempfile.gettempdir(), f"denno-beta_amd-{os.getuid()}", "_lib")):
        p = os.path.join(d, fname)
        if os.path.isfile(p):
            return p
    return None


def _compiler(kind):
    if kind == "host":
        cxx = shutil.which("g++") or shutil.which("c++")
        if not cxx:
            raise BuildError("no C++ compiler (g++) on PATH: the host core cannot be built")
        return cxx
    for c in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.isfile(c):
            return c
    raise BuildError("hipcc not found (PATH, /opt/rocm/bin): the HIP kernels cannot be built")


def spilling_kernels(compiler_output):
    """-> [(kernel, registers spilled per lane)] from the compiler's remarks on resource usage.  A kernel whose
    registers do not fit keeps some in memory and reads them back inside its loops: a product of 64 rows took 24 us
    that way where it takes 13, and no test of results sees it."""
    found, name = [], None
    for line in compiler_output.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[-R")[0].strip()
        elif "VGPRs Spill:" in line and name:
            n = int(line.split("VGPRs Spill:")[1].split("[-R")[0])
            if n > 0:
                found.append((name, n))
    return found


def _demangled(names):
    tool = shutil.which("c++filt") or "/opt/rocm/llvm/bin/llvm-cxxfilt"
    try:
        out = subprocess.run([tool], input="\n".join(names), capture_output=True, text=True, timeout=20).stdout.splitlines()
        return [o.split("(")[0].replace("void ", "") for o in out] if len(out) == len(names) else names
    except (OSError, subprocess.SubprocessError):
        return names


def compile_library(name, quiet=False):
    """Compiles `name` whether or not a built file exists; returns the path."""
    kind, sources, _ = LIBRARIES[name]
    out_dir = _lib_dir()
    final = os.path.join(out_dir, f"libdenno_{name}-{_digest(name)}.so")
    tmp = final + f".tmp{os.getpid()}"
    if not quiet:
        _say(f"compiling {name} ({', '.join(sources)}) ...")
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())   # hipcc wants a home for its caches
    # a line now and then while a long compilation runs
    done = threading.Event()

    def tick():
        while not done.wait(20.0):
            _say(f"  still compiling {name} ({time.time() - t0:.0f} s)")
    th = threading.Thread(target=tick, daemon=True)
    if not quiet:
        th.start()

    def call(cmd):
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
        if proc.returncode != 0:
            raise BuildError(f"building {name} failed ({' '.join(cmd)}):\n{proc.stdout}")
        return proc.stdout

    include = ["-I", os.path.join(_CSRC, "kernels")]
    flags = HIP_FLAGS if kind == "hip" else HOST_FLAGS
    objects = []
    try:
        if kind == "hip" and len(sources) > 1:
            # a kernel library of several source files: each compiled to an object of its own, side by side,
            # then linked (the files of the matrix products take a minute one after the other)
            objects = [f"{tmp}.{i}.o" for i in range(len(sources))]
            outs, errors = [None] * len(sources), []

            def one(i):
                try:
                    outs[i] = call([_compiler(kind)] + [f for f in flags if f != "-shared"] +
                                   ["-c", os.path.join(_CSRC, sources[i])] + include + ["-o", objects[i]])
                except Exception as e:   # raised below, after every compilation has ended
                    errors.append(e)
            workers = [threading.Thread(target=one, args=(i,)) for i in range(len(sources))]
            for w in workers:
                w.start()
            for w in workers:
                w.join()
            if errors:
                raise errors[0]
            out = "".join(outs) + call([_compiler(kind), "--offload-arch=" + HIP_ARCH, "-shared", "-fPIC"] + objects + ["-o", tmp])
        else:
            out = call([_compiler(kind)] + flags + [os.path.join(_CSRC, s) for s in sources] + include + ["-o", tmp])
    except BaseException:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise
    finally:
        done.set()
        for o in objects:
            if os.path.exists(o):
                os.remove(o)
    os.replace(tmp, final)
    for f in os.listdir(out_dir):   # built files of older sources
        if f.startswith(f"libdenno_{name}-") and f.endswith(".so") and os.path.join(out_dir, f) != final:
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    spills = spilling_kernels(out) if kind == "hip" else []
    if not quiet:
        _say(f"built {name} in {time.time() - t0:.1f} s")
        if spills:
            _say(f"  {len(spills)} kernels of {name} keep registers in memory: "
                 + "; ".join(f"{k} ({n})" for k, (_, n) in zip(_demangled([s[0] for s in spills]), spills)))
    return final


def load_library(name) -> ctypes.CDLL:
    """The loaded library; built first if no built file matches the sources."""
    with _lock:
        if name in _loaded:
            return _loaded[name]
        path = _find_built(name) or compile_library(name)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"{path} cannot be loaded: {e}") from None
        _loaded[name] = lib
        return lib


def ensure_built(names, jobs=4):
    """Compiles those of `names` that have no built file yet, side by side: a program's first call then waits for
    the longest compilation, not for their sum."""
    with _lock:
        missing = [n for n in names if n not in _loaded and _find_built(n) is None]
    if len(missing) > 1:
        build_all(missing, jobs)


def build_all(names=None, jobs=4):
    """Compiles every library (or `names`) anew, a few at a time."""
    names = list(names or LIBRARIES)
    errors, sem = [], threading.Semaphore(jobs)

    def one(n):
        with sem:
            try:
                compile_library(n)
            except Exception as e:   # collected, raised below
                errors.append(e)
    threads = [threading.Thread(target=one, args=(n,)) for n in names]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
    return names
