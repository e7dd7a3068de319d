"""Feed-forwards: the parts that work on each token alone."""
from __future__ import annotations

from .base import FEED_FORWARDS, Part
from .linear import Linear

ACTIVATION_EPILOGUES = {"gelu_tanh": "gelu_tanh", "gelu_erf": "gelu_erf"}


@FEED_FORWARDS.register("dense_mlp")
class DenseMLP(Part):
    """act(h W_up + b_up) W_down + b_down, added into the residual stream
    (crates/denno-engine/src/model/gpt2.rs:211-219).  The activation runs in the first
    product's epilogue, in 32-bit, before the rounding to the activation dtype."""
    graph_safe = True

    def __init__(self, width: int, inner: int, activation: str, up_weight: str, up_bias, down_weight: str,
                 down_bias, stored_in_out: bool = False, down_init_std: float = 0.02):
        if activation not in ACTIVATION_EPILOGUES:
            raise ValueError(f"activation {activation!r}; known: {sorted(ACTIVATION_EPILOGUES)}")
        self.width, self.inner, self.activation = width, inner, activation
        self.up = Linear(width, inner, up_weight, up_bias, stored_in_out)
        self.down = Linear(inner, width, down_weight, down_bias, stored_in_out, down_init_std)

    def param_specs(self):
        return self.up.param_specs() + self.down.param_specs()

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.up.bind(tensors)
        self.down.bind(tensors)

    def packed_input(self, n_rows):
        return self.up.packed_input(n_rows)

    def prepare_lazy_norm(self, norm):
        self.up.fold_norm(norm)

    def takes_lazy_norm(self, n_rows, norm):
        return self.up.takes_lazy_norm(n_rows, norm)

    def writes_norm_stats(self, n_rows):
        return self.down.writes_norm_stats(n_rows)

    def defers_sum(self, n_rows):
        return self.down.defers(n_rows)

    def forward(self, h, ctx, accumulate_into, stats=None, deferred=None):
        n = h.shape[0]
        f = self.up(h, out_dtype=self.runtime.act_dtype, epilogue=ACTIVATION_EPILOGUES[self.activation],
                    packed_out=self.up.few_rows(n) and self.down.packed_input(n))
        self.down(f, residual=accumulate_into, stats=stats, deferred=deferred)
