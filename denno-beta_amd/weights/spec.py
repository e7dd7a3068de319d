"""ParamSpec: what a part declares about each tensor it needs.

The model collects the specs of its parts; the loader reads exactly these names from a
checkpoint (and reports everything else), and the random initialiser draws exactly
these tensors.  A part never opens a file.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

ROLES = ("matrix", "table", "vector", "int_table")


@dataclass(frozen=True)
class ParamSpec:
    name: str                      # name in the checkpoint, without any model-wide prefix
    shape: Tuple[int, ...]         # shape as stored in the file
    role: str                      # matrix / table: compute dtype; vector: held in 32-bit; int_table: int32
    init: Tuple = ("normal", 0.0, 0.02)   # ("normal", mean, std), how random weights draw it
    transpose: bool = False        # stored [in, out]; held [out, in] (done once, at load)
    dtype_hint: Optional[str] = None      # "float32": random weights write it in 32-bit whatever the folder's dtype

    def __post_init__(self):
        if self.role not in ROLES:
            raise ValueError(f"ParamSpec {self.name}: role {self.role!r} not in {ROLES}")
        if self.transpose and len(self.shape) != 2:
            raise ValueError(f"ParamSpec {self.name}: only a matrix can be transposed")

    @property
    def held_shape(self):
        return tuple(reversed(self.shape)) if self.transpose else tuple(self.shape)
