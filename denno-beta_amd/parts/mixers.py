"""Mixers: the parts that let a token see other tokens."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import MIXERS, POSITIONS, PagedKV, Part
from .linear import Linear


@MIXERS.register("causal_attention")
class CausalSelfAttention(Part):
    """One fused projection to q | k | v, keys and values to the cache, causal softmax
    attention over the cache, output projection added into the residual stream
    (crates/denno-engine/src/model/gpt2.rs:155-208).

    n_kv_heads < n_heads: query head h reads key head h // (n_heads // n_kv_heads).
    window > 0: a query at position p reads keys p - window + 1 .. p only.
    scale multiplies the scores before the softmax.
    position: a position encoding of this layer's own, as (kind name, arguments), of the kind that
    turns queries and keys; None: the model's.
    qkv_weight_sources, qkv_bias_sources: ((file name, columns), ...) where the checkpoint stores the three
    projections as tensors of their own; qkv_weight / qkv_bias then only name the joined tensors."""
    graph_safe = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                 qkv_weight: str, qkv_bias, out_weight: str, out_bias, stored_in_out: bool = False,
                 window: int = 0, out_init_std: float = 0.02, position=None, qkv_weight_sources=None,
                 qkv_bias_sources=None):
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.scale, self.window = float(scale), int(window)
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"{n_heads} heads cannot share {n_kv_heads} key heads")
        if not 1 <= head_dim <= 256:
            raise ValueError(f"head size {head_dim}: the attention kernels take head sizes up to 256")
        self.q_width = n_heads * head_dim
        self.kv_width = n_kv_heads * head_dim
        # (a checkpoint that stores q, k and v apart names them in qkv_*_sources: joined at load, one product here)
        self.qkv = Linear(width, self.q_width + 2 * self.kv_width, qkv_weight, qkv_bias, stored_in_out,
                          weight_sources=qkv_weight_sources, bias_sources=qkv_bias_sources)
        self.out = Linear(self.q_width, width, out_weight, out_bias, stored_in_out, out_init_std)
        self.position = POSITIONS.make(position) if position is not None else None
        if self.position is not None:
            self.graph_safe = getattr(self.position, "graph_safe", False)

    def param_specs(self):
        own = self.position.param_specs() if self.position is not None else []
        return self.qkv.param_specs() + self.out.param_specs() + own

    def cache_spec(self):
        return PagedKV(self.n_kv_heads, self.head_dim, self.window)

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.qkv.bind(tensors)
        self.out.bind(tensors)
        if self.position is not None:
            self.position.bind(tensors, runtime)

    def packed_input(self, n_rows):
        return self.qkv.packed_input(n_rows)

    def prepare_lazy_norm(self, norm):
        self.qkv.fold_norm(norm)

    def takes_lazy_norm(self, n_rows, norm):
        return self.qkv.takes_lazy_norm(n_rows, norm)

    def writes_norm_stats(self, n_rows):
        return self.out.writes_norm_stats(n_rows)

    def defers_sum(self, n_rows):
        return self.out.defers(n_rows)

    def forward(self, h, ctx, cache, accumulate_into, stats=None, deferred=None):
        act = self.runtime.act_dtype
        g = ctx.groups[cache.group]
        position = self.position if self.position is not None else self.runtime.position
        if position is not None and getattr(position, "rotates", False):
            # queries and keys are turned by their positions before the keys go to the cache: the
            # product, the turn and the cache write are three steps here, not one kernel
            qkv = self.qkv(h, out_dtype=act)
            q = qkv[:, :self.q_width]
            position.rotate(q, qkv[:, self.q_width:self.q_width + self.kv_width], ctx)
            if cache.writes:
                ops.kv_write(qkv, self.q_width, self.q_width + self.kv_width, g.slot_map, cache.k, cache.v)
        elif cache.writes:
            q = self.qkv.project_qkv(h, act, g.slot_map, cache.k, cache.v, self.q_width)
        else:
            q = self.qkv(h, out_dtype=act)[:, :self.q_width]
        # the bfloat16 kernels hand their rows to the output projection packed, if it wants that
        if self.out.packed_input(h.shape[0]) and ops.attention_writes_packed(
                act, cache.k.shape[2], self.head_dim, g.single_rows, g.max_context, g.tiles_wide):
            o = ops.packed_rows(h.shape[0], self.q_width, h.device)
        else:
            o = torch.empty((h.shape[0], self.q_width), dtype=act, device=h.device)
        ops.attention(q, o, cache.k, cache.v, g.block_tables, g.tiles, self.n_heads,
                      self.scale, self.window, tiles_wide=g.tiles_wide, single_rows=g.single_rows,
                      max_context=g.max_context)
        self.out(o, residual=accumulate_into, stats=stats, deferred=deferred)
