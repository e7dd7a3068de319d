"""Block arrangements: where the norms stand around mixers and feed-forwards.

An arrangement names its parts itself: SLOTS maps each part's name in the block to its kind ("norm",
"mixer", "feed_forward").  A layer's description gives a part for every slot; the model builds them
from the parts' registries and hands them to the arrangement's constructor by those names.  The
arrangement says which of them keep caches (`mixers()`, in the order in which a LayerCall lists their
caches) and runs them (`forward(x, ctx, caches, runtime)`, `caches` in that same order)."""
from __future__ import annotations

from ..kernels import ops
from .base import ARRANGEMENTS, LazyNorm, StreamStats


@ARRANGEMENTS.register("pre_norm")
class PreNormBlock:
    """x += mixer(norm1(x)); x += ffn(norm2(x))     (crates/denno-engine/src/model/gpt2.rs:152-220)"""

    SLOTS = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ffn": "feed_forward"}

    def __init__(self, norm1, mixer, norm2, ffn):
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn

    def parts(self):
        return [self.norm1, self.mixer, self.norm2, self.ffn]

    def mixers(self):
        return [self.mixer]

    def first_norm(self):
        """The norm that reads the residual stream first in this block."""
        return self.norm1

    def after_bind(self):
        self.mixer.prepare_lazy_norm(self.norm1)
        self.ffn.prepare_lazy_norm(self.norm2)

    def forward(self, x, ctx, caches, runtime):
        cache = caches[0]
        # A norm is a kernel of its own, or, where the parts on both sides of it can (steps of few
        # rows), it runs inside them: the part before leaves what the norm needs as it adds into the
        # stream, the part after applies it in its own kernel (parts.base.StreamStats, LazyNorm).
        n = x.shape[0] if runtime.norms_inside_products else 1 << 30      # (so many rows nobody takes)
        before = runtime.stream_stats
        if before is not None and not (before.written and before.norm is self.norm1
                                       and self.mixer.takes_lazy_norm(n, self.norm1)):
            before = None
        between = (self._stats(x, self.norm2)
                   if self.mixer.writes_norm_stats(n) and self.ffn.takes_lazy_norm(n, self.norm2) else None)
        nxt = runtime.next_norm
        after = self._stats(x, nxt) if nxt is not None and self.ffn.writes_norm_stats(n) else None
        runtime.stream_stats = None
        self.mixer.forward(self._normed(self.norm1, x, self.mixer, before, runtime), ctx, cache, accumulate_into=x,
                           **({"stats": between} if between is not None else {}))
        if between is not None and not between.written:
            between = None
        self.ffn.forward(self._normed(self.norm2, x, self.ffn, between, runtime), ctx, accumulate_into=x,
                         **({"stats": after} if after is not None else {}))
        runtime.stream_stats = after if after is not None and after.written else None

    @staticmethod
    def _stats(x, norm):
        if getattr(norm, "fused_params", None) is None:
            return None
        return StreamStats(*ops.norm_stream_buffers(x.shape[0], x.shape[1], x.device), norm)

    @staticmethod
    def _normed(norm, x, part, stream, runtime):
        """The rows that `part` reads: normed here, or left to the part's own first kernel."""
        if stream is not None:
            return LazyNorm(norm, x, runtime.act_dtype, stream)
        return norm.forward(x, runtime.act_dtype, packed=part.packed_input(x.shape[0]))
