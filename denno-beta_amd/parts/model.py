"""A decoder described as data, and the model built from the description.

DecoderSpec names, layer by layer, the arrangement and the parts of each layer (for every slot
that the arrangement declares, a kind name and its arguments, looked up in the parts'
registries), and the order in which layers run: a list of LayerCall, which may name a layer
twice (its weights are shared; each call has caches of its own) or let a call read the cache
that another call writes.  What stands around the layers is described too: the token table
and a multiplier for its rows, the position encoding, the final norm, the head (tied to the token
table or a matrix of its own, with or without a bias) and what happens to its logits (a scale, a
soft cap).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import ARRANGEMENTS, KINDS, NORMS, POSITIONS, FixedState, PagedKV, Runtime
from .linear import Linear
from .positions import TokenEmbedding

PartSpec = Tuple[str, dict]   # (kind name in its registry, constructor arguments)


@dataclass
class LayerSpec:
    arrangement: str              # name in ARRANGEMENTS
    parts: Dict[str, PartSpec]    # a part for every slot that the arrangement declares (its SLOTS)


@dataclass
class LayerCall:
    layer: int                    # index into DecoderSpec.layers
    cache: Union[int, Tuple[int, ...]]   # the cache this call uses; a tuple: one for each mixer of the layer
    writes_cache: bool = True     # False: it only reads what another call wrote

    def caches(self) -> Tuple[int, ...]:
        return (self.cache,) if isinstance(self.cache, int) else tuple(self.cache)


@dataclass
class EmbeddingTable:
    """A further table [rows, width] whose rows are added to the token and position rows in the embedding kernel.
    index: which per-row integers of the step pick its rows: "tokens" or "positions" (fields of StepContext)."""
    name: str                     # checkpoint name
    rows: int
    index: str = "tokens"
    scale: float = 1.0


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
    head_bias: Optional[str] = None       # a bias added to the logits
    logit_scale: float = 1.0              # the logits times this
    logit_softcap: float = 0.0            # > 0: then cap * tanh(logit / cap)
    embedding_scale: float = 1.0          # the token table's rows times this, before the position table's
    extra_embeddings: List[EmbeddingTable] = field(default_factory=list)   # added behind them, in this order
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
        for t in spec.extra_embeddings:
            if t.index not in ("tokens", "positions"):
                raise ValueError(f"embedding table {t.name!r}: rows are picked by 'tokens' or 'positions', not {t.index!r}")
        if len(spec.extra_embeddings) > ops.EMBED_TABLES_MAX - 2:
            raise ValueError(f"{len(spec.extra_embeddings)} further embedding tables; the kernel adds up {ops.EMBED_TABLES_MAX} in all")
        self.extra_tables = {}
        self.blocks = []
        for i, ls in enumerate(spec.layers):
            if ls.arrangement not in ARRANGEMENTS:
                raise KeyError(f"no block arrangement named {ls.arrangement!r}; known: {sorted(ARRANGEMENTS)}")
            cls = ARRANGEMENTS[ls.arrangement]
            if set(ls.parts) != set(cls.SLOTS):
                raise ValueError(f"layer {i}: arrangement {ls.arrangement!r} has the parts {sorted(cls.SLOTS)}, "
                                 f"the description gives {sorted(ls.parts)}")
            self.blocks.append(cls(**{slot: KINDS[kind].make(ls.parts[slot]) for slot, kind in cls.SLOTS.items()}))
        self.final_norm = NORMS.make(spec.final_norm)
        # the head: a matrix of its own, or the token table, transposed
        self.head = Linear(spec.width, spec.vocab, spec.head_weight or spec.token_table, spec.head_bias)
        self._check_run_order()
        self.runtime = None
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in self.all_parts())

    # -- description ---------------------------------------------------------------------
    def _check_run_order(self):
        spec = self.spec
        if not spec.run_order:
            raise ValueError("run_order is empty")
        n_caches = max(max(c.caches()) for c in spec.run_order) + 1
        writer = [None] * n_caches        # cache -> (call, the cache's need) of the call that writes it
        for i, c in enumerate(spec.run_order):
            if not 0 <= c.layer < len(spec.layers):
                raise ValueError(f"run_order[{i}] names layer {c.layer}; there are {len(spec.layers)}")
            mixers = self.blocks[c.layer].mixers()
            if len(c.caches()) != len(mixers):
                raise ValueError(f"run_order[{i}] names {len(c.caches())} caches; layer {c.layer} has {len(mixers)} mixers")
            for cache, mixer in zip(c.caches(), mixers):
                cs = mixer.cache_spec()
                if cache < 0:
                    raise ValueError(f"run_order[{i}] names cache {cache}")
                if c.writes_cache:
                    if writer[cache] is not None:
                        raise ValueError(f"run_order[{i}] writes cache {cache}, which run_order[{writer[cache][0]}] writes")
                    writer[cache] = (i, cs)
                else:
                    if writer[cache] is None:
                        raise ValueError(f"run_order[{i}] reads cache {cache} before any call has written it")
                    if writer[cache][1] != cs:
                        raise ValueError(f"run_order[{i}] reads cache {cache}, whose writer keeps another kind of cache")
        if any(w is None for w in writer):
            raise ValueError("a cache index is never written")
        self.n_caches = n_caches
        self.cache_specs = [w[1] for w in writer]

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
        for t in self.spec.extra_embeddings:
            if t.name in seen:
                raise ValueError(f"two parts claim the tensor {t.name!r}")
            seen.add(t.name)
            specs.append(ParamSpec(t.name, (t.rows, self.spec.width), "table", ("normal", 0.0, 0.02)))
        specs += [s for s in self.head.param_specs() if s.name not in seen]     # (a tied head's weight is the table's)
        return specs

    # -- binding -------------------------------------------------------------------------
    def bind(self, tensors: Dict[str, torch.Tensor], runtime: Runtime):
        self.runtime = runtime
        runtime.position = self.position          # mixers ask it to turn their queries and keys, if it does that
        for p in self.all_parts():
            p.bind(tensors, runtime)
        self.head.bind(tensors)
        self.extra_tables = {t.name: tensors[t.name] for t in self.spec.extra_embeddings}
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
        if not self.spec.extra_embeddings:
            ops.embed(ctx.tokens, ctx.positions, self.embedding.weight, self.position.table(), x,
                      token_scale=self.spec.embedding_scale)
        else:
            parts = [(self.embedding.weight, ctx.tokens, self.spec.embedding_scale)]
            if self.position.table() is not None:
                parts.append((self.position.table(), ctx.positions, 1.0))
            parts += [(self.extra_tables[t.name], getattr(ctx, t.index), t.scale) for t in self.spec.extra_embeddings]
            ops.embed_sum(parts, x)
        rt.stream_stats = rt.stream_deferred = None      # nobody has left anything for a norm of these rows yet
        order = self.spec.run_order
        for i, call in enumerate(order):
            nxt = self.blocks[order[i + 1].layer] if i + 1 < len(order) else None
            rt.next_norm = nxt.first_norm() if nxt is not None and hasattr(nxt, "first_norm") else None
            rt.next_takes_deferred = nxt is not None and getattr(nxt, "takes_deferred", False)
            block = self.blocks[call.layer]
            if rt.stream_deferred is not None and not getattr(block, "takes_deferred", False):
                rt.stream_deferred.flush(x)         # (an arrangement that knows nothing of sums left for its norm)
                rt.stream_deferred = None
            block.forward(x, ctx, [cache.view(c, call.writes_cache) for c in call.caches()], rt)
        if rt.stream_deferred is not None:
            rt.stream_deferred.flush(x)
        rt.stream_stats = rt.next_norm = rt.stream_deferred = None
        rt.next_takes_deferred = False
        if ctx.R == 0:
            return torch.empty((0, self.spec.vocab), dtype=torch.float32, device=rt.device)
        h = self.final_norm.forward(x, rt.act_dtype, rows=ctx.logit_rows, packed=self.head.packed_input(ctx.R))
        logits = self.head(h, out_dtype=torch.float32)
        if self.spec.logit_scale != 1.0 or self.spec.logit_softcap > 0:
            ops.logits_post(logits, self.spec.logit_scale, self.spec.logit_softcap)
        return logits
