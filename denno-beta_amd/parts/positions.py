"""Position encodings and the token table.

A position encoding acts in one of two places: it gives a table that the embedding stage adds
to the token rows (`table()`), or it turns queries and keys inside a mixer (`rotates = True` and
`rotate(q, k, ctx)`, which changes q [T, heads * dh] and k [T, kv heads * dh] in place, rows
ctx.positions; a mixer that keeps keys then writes the turned keys to its cache).  One that does
not act in a place returns None there / has `rotates = False`.
"""
from __future__ import annotations

from ..weights.spec import ParamSpec
from .base import POSITIONS, Part


class TokenEmbedding(Part):
    """The token table [vocab, width]; also the head's weight when the head is tied."""
    graph_safe = True

    def __init__(self, vocab: int, width: int, name: str):
        self.vocab, self.width, self.name = vocab, width, name

    def param_specs(self):
        return [ParamSpec(self.name, (self.vocab, self.width), "table", ("normal", 0.0, 0.02))]

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.weight = tensors[self.name]


@POSITIONS.register("learned_absolute")
class LearnedAbsolutePositions(Part):
    """x[i] += wpe[position_i]                    (crates/denno-engine/src/model/gpt2.rs:142-150)"""
    graph_safe = True
    rotates = False

    def __init__(self, n_positions: int, width: int, name: str):
        self.n_positions, self.width, self.name = n_positions, width, name

    def param_specs(self):
        return [ParamSpec(self.name, (self.n_positions, self.width), "table", ("normal", 0.0, 0.02))]

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.weight = tensors[self.name]

    def table(self):
        return self.weight

    def rotate(self, q, k, ctx):
        return q, k


@POSITIONS.register("none")
class NoPositions(Part):
    graph_safe = True
    rotates = False

    def __init__(self):
        pass

    def table(self):
        return None

    def rotate(self, q, k, ctx):
        return q, k
