"""Hand-written HIP kernels for gfx950 (sources: ../csrc/kernels) behind `ops`."""
from . import ops

__all__ = ["ops"]
