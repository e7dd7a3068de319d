"""Runs the engine's host logic on the CPU by putting the plain references of
`kernel_refs` in the kernels' place.  For tests only: the product has no such path."""
from __future__ import annotations

import contextlib

import kernel_refs
from denno_beta_amd.kernels import ops

_NAMES = ["embed", "embed_sum", "logits_post", "layernorm", "kv_write", "cast", "linear", "linear_qkv", "linear_norm_out", "linear_norm_in", "attention", "sample", "sample_top", "sample_full", "penalties", "history_append"]


@contextlib.contextmanager
def emulated_kernels():
    saved = {n: getattr(ops, n) for n in _NAMES}
    try:
        for n in _NAMES:
            setattr(ops, n, getattr(kernel_refs, n))
        yield
    finally:
        for n, f in saved.items():
            setattr(ops, n, f)
