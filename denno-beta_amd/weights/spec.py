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
    # A tensor that the checkpoint stores in pieces (a fused projection whose q, k and v are tensors of their own):
    # ((file name, size along concat_dim), ...) in the order in which they are joined; `name` is then the held
    # tensor's name only and appears in no file.  The sizes add up to shape[concat_dim] (of the stored layout).
    sources: Optional[Tuple[Tuple[str, int], ...]] = None
    concat_dim: int = 0

    def __post_init__(self):
        if self.role not in ROLES:
            raise ValueError(f"ParamSpec {self.name}: role {self.role!r} not in {ROLES}")
        if self.transpose and len(self.shape) != 2:
            raise ValueError(f"ParamSpec {self.name}: only a matrix can be transposed")
        if self.sources is not None:
            if not 0 <= self.concat_dim < len(self.shape):
                raise ValueError(f"ParamSpec {self.name}: concat_dim {self.concat_dim} outside its {len(self.shape)} dimensions")
            if not self.sources or sum(n for _, n in self.sources) != self.shape[self.concat_dim]:
                raise ValueError(f"ParamSpec {self.name}: its sources' sizes {[n for _, n in self.sources]} do not add up to "
                                 f"{self.shape[self.concat_dim]}")

    def pieces(self):
        """[(file name, stored shape)] of the file tensors that make this one: itself, or its sources."""
        if self.sources is None:
            return [(self.name, tuple(self.shape))]
        out = []
        for fname, n in self.sources:
            shape = list(self.shape)
            shape[self.concat_dim] = n
            out.append((fname, tuple(shape)))
        return out

    @property
    def held_shape(self):
        return tuple(reversed(self.shape)) if self.transpose else tuple(self.shape)
