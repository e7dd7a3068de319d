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
  arrangement      ARRANGEMENTS    forward(x, ctx, cache): how norms, mixer and feed-forward stand in a block

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
    """A mixer that keeps keys and values of `window` last positions (0: all) in pages."""
    n_kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class FixedState:
    """A mixer that keeps a state of fixed size per request: a tensor of `shape` and `dtype`,
    zero when a request starts."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


@dataclass
class Runtime:
    """What parts need to know about the engine they are bound into.  `position` is the model's
    position encoding (set by the model before it binds its parts): a mixer asks it to turn its
    queries and keys if it is of the kind that does (`rotates`)."""
    act_dtype: torch.dtype
    device: torch.device
    position: Optional["Part"] = None


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

    # helpers ---------------------------------------------------------------
    def _take(self, tensors, name):
        return tensors[name]


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
