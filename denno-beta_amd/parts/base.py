"""What every part is: a description (sizes and constants as constructor arguments), the
tensors it needs (ParamSpecs), and a forward over the batch of one step.

No part knows which model it is in.  A part's constructor takes plain numbers and names;
`param_specs()` lists its tensors under the names the architecture gave it; `bind()` receives
them on the device; `forward` runs on the rows of one step.

Kinds of part and their registries:

  mixer            MIXERS          forward(h, ctx, cache, accumulate_into) ; cache_spec()
  feed-forward     FEED_FORWARDS   forward(h, ctx, accumulate_into)
  norm             NORMS           forward(x, out_dtype, rows=None) -> tensor
  position code    POSITIONS       table() for the embedding stage, rotate(q, k, ctx) for mixers
  arrangement      ARRANGEMENTS    SLOTS names its parts and their kinds; forward(x, ctx, caches, runtime): how
                                   norms, mixers and feed-forwards stand in a block

`h` is [T, width] in the activation dtype; `x` and `accumulate_into` are the 32-bit residual
stream [T, width], which mixers and feed-forwards add their result to in place (the sum is
made in 32-bit inside the last kernel).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from ..weights.spec import ParamSpec


@dataclass(frozen=True)
class PagedKV:
    """A mixer that keeps keys and values of `window` last positions (0: all) in pages.
    dtype: what the pages hold ("bfloat16", "float32"); None: the engine's activation dtype.
    head_dim is the width of a key; value_dim that of a value (None: the same).  The pools are laid out for
    both ([.., Hkv, page, head_dim] and [.., Hkv, value_dim, page]); the attention kernels of this package
    take equal widths only and say so when they are asked for others (kernels.ops.attention), so a mixer whose
    values are wider or narrower than its keys brings a kernel of its own for the same pools."""
    n_kv_heads: int
    head_dim: int
    window: int = 0
    dtype: Optional[str] = None
    value_dim: Optional[int] = None

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class FixedState:
    """A mixer that keeps a state of fixed size per request: a tensor of `shape` and `dtype`,
    zero when a request starts."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


@dataclass
class Runtime:
    """What parts need to know about the engine they are bound into.  `position` is the model's
    position encoding (set by the model before it binds its parts): a mixer that names no position
    encoding of its own asks this one to turn its queries and keys, if it is of the kind that does
    (`rotates`)."""
    act_dtype: torch.dtype
    device: torch.device
    position: Optional["Part"] = None
    norms_inside_products: bool = True     # EngineOptions.norms_inside_products
    # what the last part that added into the residual stream left for the norm after it (StreamStats),
    # or None; the model clears it where the stream changes in any other way
    stream_stats: Optional["StreamStats"] = None
    # the norm that will read the stream first after the block that runs now (set by the model), or None
    next_norm: Optional["Part"] = None
    next_takes_deferred: bool = False      # the block that runs next takes what is left in stream_deferred (set by the model)
    deferred_sums: bool = True             # EngineOptions.deferred_sums
    # a product's sum that is not in the stream yet (DeferredSum): the next norm's kernel adds it, or the model does
    stream_deferred: Optional["DeferredSum"] = None


class Part:
    """Base of all parts.

    graph_safe: the part's forward reads the step's tables on the device only (no loop over
    requests on the host, no size taken from a table's contents), so a decode step with it can be
    captured once as a HIP graph and replayed over new tables."""
    graph_safe = False

    def param_specs(self) -> List[ParamSpec]:
        return []

    def bind(self, tensors: Dict[str, torch.Tensor], runtime: Runtime) -> None:
        self.runtime = runtime

    def packed_input(self, n_rows: int) -> bool:
        """A mixer or feed-forward whose first product takes packed rows (kernels.ops.PackedMatrix)
        for a step of n_rows rows says so here; the block then asks the norm before it for them.
        The default, a tensor [rows, width], is always right."""
        return False

    def prepare_lazy_norm(self, norm) -> None:
        """Called once, after binding, with the norm that stands before this part in its block: a part
        that can run that norm inside its own first kernel makes ready for it here."""

    def takes_lazy_norm(self, n_rows: int, norm) -> bool:
        """A mixer or feed-forward whose first kernel can run `norm` itself for a step of n_rows rows,
        given what the part before left (StreamStats), says so here; the block then hands it a
        LazyNorm in place of the normed rows.  The default, normed rows, is always right."""
        return False

    def defers_sum(self, n_rows: int) -> bool:
        """A mixer or feed-forward whose last product, for a step of n_rows rows, can leave its sum for the norm
        that reads the stream next to add (DeferredSum); its forward then takes `deferred=` (an empty DeferredSum
        that it may fill instead of adding into the stream)."""
        return False

    def writes_norm_stats(self, n_rows: int) -> bool:
        """A mixer or feed-forward whose last kernel, as it adds into the residual stream, can leave
        the statistics for the norm after it; its forward then takes `stats=` (a StreamStats)."""
        return False

    # helpers ---------------------------------------------------------------
    def _take(self, tensors, name):
        return tensors[name]


class StreamStats:
    """What one norm of the residual stream's rows needs, left by the kernel that last added into
    the stream: the rows times that norm's weight, rounded to bfloat16, and per row and block of 16
    columns the mean and the sum of squared distances from it (kernels.ops.linear_norm_out /
    linear_norm_in).  `norm` is the norm it was made for: nobody else may use it."""

    def __init__(self, copy, stats, norm):
        self.copy, self.stats, self.norm = copy, stats, norm
        self.written = False


class DeferredSum:
    """What a part's last product would have added into the residual stream, left for the kernel of the norm that
    reads the stream next: the product's sums by shares of K, 32-bit [shares, rows, width], and its bias.  A norm
    with `adds_deferred = True` takes it as `forward(..., deferred=)` and leaves the stream updated; anybody else
    has it added first (`flush`)."""

    def __init__(self):
        self.part = self.bias = None

    @property
    def filled(self):
        return self.part is not None

    def fill(self, part, bias):
        self.part, self.bias = part, bias

    def flush(self, x):
        from ..kernels import ops
        if self.filled:
            ops.join(self.part, self.bias, x)
            self.part = self.bias = None


class LazyNorm:
    """Rows that are not normed yet: a norm, the residual stream it is to read and the statistics
    that were left for it.  Whoever receives it runs the norm inside its own kernel or asks for
    the rows (`rows()`)."""

    def __init__(self, norm, x, dtype, stream: StreamStats):
        self.norm, self.x, self.dtype, self.stream = norm, x, dtype, stream
        self.shape, self.device = x.shape, x.device

    def rows(self, packed=False):
        return self.norm.forward(self.x, self.dtype, packed=packed)


class Registry(dict):
    def __init__(self, kind):
        super().__init__()
        self.kind = kind

    def register(self, name):
        def deco(cls):
            self[name] = cls
            cls.kind_name = name
            return cls
        return deco

    def make(self, spec):
        """spec: (kind name, kwargs)."""
        name, kwargs = spec
        if name not in self:
            raise KeyError(f"no {self.kind} named {name!r}; known: {sorted(self)}")
        return self[name](**kwargs)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
ARRANGEMENTS = Registry("block arrangement")
# the kinds that an arrangement's SLOTS may name
KINDS = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS}
