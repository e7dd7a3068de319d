"""Block arrangements: where the norms stand around a mixer and a feed-forward."""
from __future__ import annotations

from .base import ARRANGEMENTS


@ARRANGEMENTS.register("pre_norm")
class PreNormBlock:
    """x += mixer(norm1(x)); x += ffn(norm2(x))     (crates/denno-engine/src/model/gpt2.rs:152-220)"""

    def __init__(self, norm1, mixer, norm2, ffn):
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn

    def parts(self):
        return [self.norm1, self.mixer, self.norm2, self.ffn]

    def forward(self, x, ctx, cache, runtime):
        n = x.shape[0]
        h = self.norm1.forward(x, runtime.act_dtype, packed=self.mixer.packed_input(n))
        self.mixer.forward(h, ctx, cache, accumulate_into=x)
        h = self.norm2.forward(x, runtime.act_dtype, packed=self.ffn.packed_input(n))
        self.ffn.forward(h, ctx, accumulate_into=x)
