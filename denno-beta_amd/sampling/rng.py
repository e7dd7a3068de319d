"""A counter-based generator: the n-th uniform number of a request is a function of
(seed, n) only, so a request's samples depend neither on the batch nor on preemption.
The reference seeds one `StdRng` per request (crates/denno-engine/src/sampler.rs:339-342);
its stream is not reproduced."""
from __future__ import annotations

import os

_M = (1 << 64) - 1


def _mix(z: int) -> int:
    # splitmix64's finaliser
    z = (z + 0x9E3779B97F4A7C15) & _M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M
    return z ^ (z >> 31)


def uniform(seed: int, n: int) -> float:
    """The n-th number in [0, 1) of the stream `seed`: 24 random bits, exact in 32-bit."""
    return (_mix(_mix(seed & _M) ^ ((n * 0xD1342543DE82EF95) & _M)) >> 40) / float(1 << 24)


def entropy_seed() -> int:
    return int.from_bytes(os.urandom(8), "little")
