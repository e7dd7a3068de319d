"""A decoder described as data, and the model built from the description.

DecoderSpec names, layer by layer, the arrangement and the parts of each layer (a kind name
and its arguments, looked up in the parts' registries), and the order in which layers run:
a list of LayerCall, which may name a layer twice (its weights are shared; each call has a
cache of its own) or let a call read the cache that another call writes.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, FixedState, PagedKV, Runtime
from .linear import Linear
from .positions import TokenEmbedding

PartSpec = Tuple[str, dict]   # (kind name in its registry, constructor arguments)


@dataclass
class LayerSpec:
    arrangement: str
    norm1: PartSpec
    mixer: PartSpec
    norm2: PartSpec
    ffn: PartSpec


@dataclass
class LayerCall:
    layer: int                    # index into DecoderSpec.layers
    cache: int                    # index of the cache this call uses
    writes_cache: bool = True     # False: it only reads what another call wrote


@dataclass
class DecoderSpec:
    vocab: int
    width: int
    max_positions: int
    token_table: str              # checkpoint name of the token table
    position: PartSpec
    layers: List[LayerSpec]
    run_order: List[LayerCall]
    final_norm: PartSpec
    head_weight: Optional[str] = None     # None: the head is the token table, transposed
    eos_token_ids: Tuple[int, ...] = ()
    # how checkpoints of this architecture name things
    name_prefixes: Tuple[str, ...] = ("",)
    ignore_tensors: Tuple[str, ...] = ()
    tied_tensors: Dict[str, str] = field(default_factory=dict)

    def instantiate(self) -> "DecoderModel":
        return DecoderModel(self)

    def param_specs(self) -> List[ParamSpec]:
        return self.instantiate().param_specs()


@dataclass
class CacheView:
    """What a mixer sees of the cache during one call."""
    group: int                    # index into ctx.groups
    writes: bool
    k: Optional[torch.Tensor] = None       # paged: [n_pages, Hkv, page_size, dh] of this call's cache
    v: Optional[torch.Tensor] = None       #        [n_pages, Hkv, dh, page_size]
    state: Optional[torch.Tensor] = None   # fixed state: [n_slots, *shape]


class DecoderModel:
    def __init__(self, spec: DecoderSpec):
        self.spec = spec
        self.embedding = TokenEmbedding(spec.vocab, spec.width, spec.token_table)
        self.position = POSITIONS.make(spec.position)
        self.blocks = []
        for ls in spec.layers:
            if ls.arrangement not in ARRANGEMENTS:
                raise KeyError(f"no block arrangement named {ls.arrangement!r}; known: {sorted(ARRANGEMENTS)}")
            self.blocks.append(ARRANGEMENTS[ls.arrangement](
                NORMS.make(ls.norm1), MIXERS.make(ls.mixer), NORMS.make(ls.norm2), FEED_FORWARDS.make(ls.ffn)))
        self.final_norm = NORMS.make(spec.final_norm)
        self.head = None if spec.head_weight is None else Linear(spec.width, spec.vocab, spec.head_weight, None)
        self._check_run_order()
        self.runtime = None
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.all_parts())

    # -- description ---------------------------------------------------------------------
    def _check_run_order(self):
        spec = self.spec
        if not spec.run_order:
            raise ValueError("run_order is empty")
        n_caches = max(c.cache for c in spec.run_order) + 1
        writer = [None] * n_caches
        for i, c in enumerate(spec.run_order):
            if not 0 <= c.layer < len(spec.layers):
                raise ValueError(f"run_order[{i}] names layer {c.layer}; there are {len(spec.layers)}")
            cs = self.blocks[c.layer].mixer.cache_spec()
            if c.writes_cache:
                if writer[c.cache] is not None:
                    raise ValueError(f"run_order[{i}] writes cache {c.cache}, which run_order[{writer[c.cache]}] writes")
                writer[c.cache] = i
            else:
                if writer[c.cache] is None:
                    raise ValueError(f"run_order[{i}] reads cache {c.cache} before any call has written it")
                if self.blocks[spec.run_order[writer[c.cache]].layer].mixer.cache_spec() != cs:
                    raise ValueError(f"run_order[{i}] reads cache {c.cache}, whose writer keeps another kind of cache")
        if any(w is None for w in writer):
            raise ValueError("a cache index is never written")
        self.n_caches = n_caches
        self.cache_specs = [self.blocks[spec.run_order[w].layer].mixer.cache_spec() for w in writer]

    def all_parts(self):
        parts = [self.embedding, self.position]
        for b in self.blocks:
            parts += b.parts()
        parts.append(self.final_norm)
        return parts

    def param_specs(self) -> List[ParamSpec]:
        specs, seen = [], set()
        for p in self.all_parts():
            for s in p.param_specs():
                if s.name in seen:
                    raise ValueError(f"two parts claim the tensor {s.name!r}")
                seen.add(s.name)
                specs.append(s)
        if self.head is not None:
            specs += self.head.param_specs()
        return specs

    # -- binding -------------------------------------------------------------------------
    def bind(self, tensors: Dict[str, torch.Tensor], runtime: Runtime):
        self.runtime = runtime
        runtime.position = self.position          # mixers ask it to turn their queries and keys, if it does that
        for p in self.all_parts():
            p.bind(tensors, runtime)
        if self.head is not None:
            self.head.bind(tensors)
        else:
            self.head = Linear(self.spec.width, self.spec.vocab, self.spec.token_table, None)
            self.head.bind(tensors)
        for b in self.blocks:
            after = getattr(b, "after_bind", None)     # an arrangement may make its parts ready for each other
            if after is not None:
                after()
        return self

    def weight_bytes(self, tensors=None):
        """Bytes of every weight a step reads once (the position table aside: a step reads T rows of it)."""
        total, seen = 0, set()
        def add(t):
            nonlocal total
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        for b in self.blocks:
            for p in b.parts():
                for v in vars(p).values():
                    if isinstance(v, Linear):
                        add(v.weight), add(v.bias)
                    elif isinstance(v, torch.Tensor):
                        add(v)
        add(self.head.weight)
        add(getattr(self.final_norm, "weight", None)), add(getattr(self.final_norm, "bias", None))
        return total

    # -- the forward pass over one step's rows -------------------------------------------
    def forward(self, ctx, cache) -> torch.Tensor:
        """ctx: engine.batch.StepContext; cache: cache.storage.CacheStorage.
        -> 32-bit logits [R, vocab] at ctx.logit_rows."""
        rt = self.runtime
        x = torch.empty((ctx.T, self.spec.width), dtype=torch.float32, device=rt.device)
        ops.embed(ctx.tokens, ctx.positions, self.embedding.weight, self.position.table(), x)
        rt.stream_stats = None      # nobody has left anything for a norm of these rows yet
        order = self.spec.run_order
        for i, call in enumerate(order):
            nxt = self.blocks[order[i + 1].layer] if i + 1 < len(order) else None
            rt.next_norm = nxt.first_norm() if nxt is not None and hasattr(nxt, "first_norm") else None
            self.blocks[call.layer].forward(x, ctx, cache.view(call.cache, call.writes_cache), rt)
        rt.stream_stats = rt.next_norm = None
        if ctx.R == 0:
            return torch.empty((0, self.spec.vocab), dtype=torch.float32, device=rt.device)
        h = self.final_norm.forward(x, rt.act_dtype, rows=ctx.logit_rows, packed=self.head.packed_input(ctx.R))
        return self.head(h, out_dtype=torch.float32)
