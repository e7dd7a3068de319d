"""EngineOptions: everything about how the engine runs that is not the model.

The reference spreads these over command-line flags and DENNO_* environment
variables (crates/denno-engine/src/engine.rs:147-186); here they are one typed
record and no environment variable changes behaviour.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

DTYPES = ("bfloat16", "float32")
KV_POLICIES = ("preempt", "reserve")


@dataclass
class EngineOptions:
    dtype: str = "bfloat16"            # "bfloat16": serving precision; "float32": true 32-bit everywhere
    page_size: int = 16                # tokens in a page of the cache
    cache_tokens: Optional[int] = None  # size of every paged pool in tokens; None: max_live * max positions
    max_live: int = 64                 # most requests that hold cache at a time (state slots)
    max_batch_tokens: int = 2048       # token budget of one step
    prefill_chunk: int = 512           # longest portion of one prompt in one step
    kv_policy: str = "preempt"         # what happens when pages run out: see engine/scheduler.py
    device: str = "cuda:0"
    use_graphs: bool = True            # replay pure-decode steps from captured HIP graphs
    graph_portions: bool = True        # steps of up to 512 rows that hold prompt portions are captured too, a bucket at its second step (engine/graphs.py)
    run_ahead: bool = True             # launch the next decode step before the host has read this one's tokens (engine/engine.py)
    seed: Optional[int] = None         # default seed of requests that bring none
    deferred_sums: bool = True         # steps of 65 to 256 rows: a product into the stream with few columns leaves its sum for the next norm's kernel (parts/blocks.py)
    norms_inside_products: bool = True  # steps of few rows: a norm between two products runs inside them (parts/blocks.py)

    def validate(self):
        if self.dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {DTYPES}, got {self.dtype!r}")
        if self.kv_policy not in KV_POLICIES:
            raise ValueError(f"kv_policy must be one of {KV_POLICIES}, got {self.kv_policy!r}")
        if self.page_size < 1:
            raise ValueError("page_size must be >= 1")
        if self.max_live < 1 or self.max_batch_tokens < 1 or self.prefill_chunk < 1:
            raise ValueError("max_live, max_batch_tokens and prefill_chunk must be >= 1")
        return self
