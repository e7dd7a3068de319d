"""ModelRunner: a model bound to its weights and its cache, and the one step function.

`step(entries)` runs the tokens it is given, as one batch, from the cache that earlier steps
left, and returns 32-bit logits at the wanted places.  It is what generation, the scheduler's
engine and trace replay all call.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheStorage
from ..config import EngineOptions, load_config
from ..parts import Runtime
from ..weights import draw_all, load_checkpoint
from .batch import StepEntry, build_context

_ACT = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class ModelRunner:
    def __init__(self, spec, tensors, options: EngineOptions, config=None):
        options.validate()
        self.spec, self.options, self.config = spec, options, config
        self.device = torch.device(options.device)
        self.runtime = Runtime(act_dtype=_ACT[options.dtype], device=self.device,
                               norms_inside_products=options.norms_inside_products,
                               deferred_sums=options.deferred_sums)
        model = spec.instantiate()
        if self.device.type == "cuda":
            # what this model needs is compiled now, side by side, if it is not built yet (else each library
            # would be compiled at its first call, one after the other)
            from ..build import ensure_built
            from ..parts.base import PagedKV
            paged = any(isinstance(cs, PagedKV) for cs in model.cache_specs)
            ensure_built(["host", "elementwise", "gemm"] + (["attention"] if paged else []))
        self.model = model.bind(tensors, self.runtime)
        cache_tokens = options.cache_tokens or options.max_live * spec.max_positions
        self.cache = CacheStorage(self.model.cache_specs, kv_dtype=self.runtime.act_dtype,
                                  page_size=options.page_size, cache_tokens=cache_tokens,
                                  max_live=options.max_live, device=self.device)
        self.notes: List[str] = []
        self.steps_run = 0
        self.graphs = None
        if options.use_graphs and self.device.type == "cuda":
            from .graphs import DecodeGraphs
            self.graphs = DecodeGraphs(self)

    # -- construction --------------------------------------------------------------------
    @classmethod
    def from_folder(cls, model_dir: str, options: EngineOptions, cast_matrices: bool = False):
        arch, cfg = load_config(model_dir)
        spec = arch.build(cfg)
        notes: List[str] = []
        tensors = load_checkpoint(model_dir, spec.param_specs(), engine_dtype=options.dtype,
                                  device=torch.device(options.device), cast_matrices=cast_matrices,
                                  prefixes=spec.name_prefixes, ignore=spec.ignore_tensors,
                                  tied=spec.tied_tensors, notes=notes)
        r = cls(spec, tensors, options, cfg)
        r.notes = notes
        return r

    @classmethod
    def from_random(cls, config: dict, seed: int, options: EngineOptions, stored: Optional[str] = None):
        """Random weights drawn on the device, as a folder written in `stored` precision
        (default: the engine's) would load."""
        from ..config import resolve_architecture
        arch = resolve_architecture(config)
        cfg = arch.config_cls.from_dict(config)
        spec = arch.build(cfg)
        tensors = draw_all(spec.param_specs(), seed, engine_dtype=options.dtype,
                           device=torch.device(options.device), stored=stored or options.dtype)
        return cls(spec, tensors, options, cfg)

    # -- requests ------------------------------------------------------------------------
    def start_request(self, rid: int) -> int:
        return self.cache.start_request(rid)

    def end_request(self, rid: int) -> bool:
        return self.cache.manager.release(rid)

    def has_request(self, rid: int) -> bool:
        return self.cache.manager.has(rid)

    def runs_ahead(self) -> bool:
        """Whether a step of single tokens can take its tokens from the device (it is replayed from a graph)."""
        return self.graphs is not None and self.model.graph_safe

    # -- the step ------------------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], device_tokens=None, borrow=False) -> torch.Tensor:
        """-> logits [R, vocab], 32-bit, on the device: the wanted places in the order of the
        entries and of each entry's `want`.  On return the cache holds the entries' tokens.
        device_tokens: for a step of single tokens that captured graphs run (`runs_ahead`): the tokens as
        an int32 tensor on the device, where the host does not know them yet.
        borrow: the logits may be a buffer that a later step overwrites (a replayed graph's own output): for a
        caller that is done with them, on this stream, before its next step."""
        entries = list(entries)
        if not entries:
            return torch.empty((0, self.spec.vocab), dtype=torch.float32, device=self.device)
        if self.graphs is not None and self.graphs.takes(entries):
            self.steps_run += 1
            return self.graphs.step(entries, device_tokens, borrow)
        if device_tokens is not None:
            raise ValueError("device_tokens: only a step of single tokens that captured graphs run takes them")
        if self.graphs is not None and self.graphs.takes_portions(entries):
            self.steps_run += 1
            return self.graphs.step_portions(entries, borrow)
        ctx = build_context(entries, self.cache, self.spec.vocab, self.spec.max_positions, self.device)
        logits = self.model.forward(ctx, self.cache)
        self.cache.manager.commit_step(
            np.asarray(ctx.rids, dtype=np.int64),
            np.asarray([start + len(e.tokens) for e, start in zip(entries, ctx.host_first_pos)], dtype=np.int32))
        self.steps_run += 1
        return logits
