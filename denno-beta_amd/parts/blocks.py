"""Block arrangements: where the norms stand around mixers and feed-forwards.

An arrangement names its parts itself: SLOTS maps each part's name in the block to its kind ("norm",
"mixer", "feed_forward").  A layer's description gives a part for every slot; the model builds them
from the parts' registries and hands them to the arrangement's constructor by those names.  The
arrangement says which of them keep caches (`mixers()`, in the order in which a LayerCall lists their
caches) and runs them (`forward(x, ctx, caches, runtime)`, `caches` in that same order)."""
from __future__ import annotations

from ..kernels import ops
from .base import ARRANGEMENTS, DeferredSum, LazyNorm, StreamStats


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

    takes_deferred = True     # its first norm adds what the block before left in Runtime.stream_deferred

    def forward(self, x, ctx, caches, runtime):
        cache = caches[0]
        # A product into the stream may leave its sum for the kernel of the norm behind it (steps of 65 to 256
        # rows, few columns: parts.base.DeferredSum): the part before a norm is offered an empty one, the norm gets
        # what was put there; across blocks it travels in runtime.stream_deferred.
        came = runtime.stream_deferred
        runtime.stream_deferred = None
        can = runtime.deferred_sums
        mid = DeferredSum() if can and getattr(self.norm2, "adds_deferred", False) and self.mixer.defers_sum(x.shape[0]) else None
        end = (DeferredSum() if can and getattr(runtime.next_norm, "adds_deferred", False) and runtime.next_takes_deferred
               and self.ffn.defers_sum(x.shape[0]) else None)
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
        self.mixer.forward(self._normed(self.norm1, x, self.mixer, before, runtime, came), ctx, cache, accumulate_into=x,
                           **({"stats": between} if between is not None else {}),
                           **({"deferred": mid} if mid is not None else {}))
        if between is not None and not between.written:
            between = None
        self.ffn.forward(self._normed(self.norm2, x, self.ffn, between, runtime, mid), ctx, accumulate_into=x,
                         **({"stats": after} if after is not None else {}),
                         **({"deferred": end} if end is not None else {}))
        runtime.stream_stats = after if after is not None and after.written else None
        runtime.stream_deferred = end if end is not None and end.filled else None

    @staticmethod
    def _stats(x, norm):
        if getattr(norm, "fused_params", None) is None:
            return None
        return StreamStats(*ops.norm_stream_buffers(x.shape[0], x.shape[1], x.device), norm)

    @staticmethod
    def _normed(norm, x, part, stream, runtime, deferred=None):
        """The rows that `part` reads: normed here, or left to the part's own first kernel.  deferred: a sum that
        is not in the stream yet: the norm's kernel adds it, or it is added first."""
        if deferred is not None and deferred.filled:
            if getattr(norm, "adds_deferred", False) and stream is None:
                return norm.forward(x, runtime.act_dtype, packed=part.packed_input(x.shape[0]), deferred=deferred)
            deferred.flush(x)
        if stream is not None:
            return LazyNorm(norm, x, runtime.act_dtype, stream)
        return norm.forward(x, runtime.act_dtype, packed=part.packed_input(x.shape[0]))
