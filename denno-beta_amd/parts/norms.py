"""Norms."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import NORMS, Part


@NORMS.register("layernorm")
class LayerNorm(Part):
    """(x - mean) / sqrt(var + eps) * weight + bias, statistics and affine in 32-bit
    (crates/denno-engine/src/tensor.rs:1101-1112)."""
    graph_safe = True

    def __init__(self, width: int, eps: float, weight_name: str, bias_name=None):
        self.width, self.eps = width, eps
        self.weight_name, self.bias_name = weight_name, bias_name

    def param_specs(self):
        specs = [ParamSpec(self.weight_name, (self.width,), "vector", ("normal", 1.0, 0.02))]
        if self.bias_name:
            specs.append(ParamSpec(self.bias_name, (self.width,), "vector", ("normal", 0.0, 0.01)))
        return specs

    def bind(self, tensors, runtime):
        super().bind(tensors, runtime)
        self.weight = tensors[self.weight_name]
        self.bias = tensors[self.bias_name] if self.bias_name else None

    def fused_params(self):
        """What a kernel that runs this norm itself needs (parts.base.LazyNorm)."""
        return ("layernorm", self.weight, self.bias, self.eps)

    adds_deferred = True      # forward(..., deferred=): its kernel first adds a product's sum into the rows (parts.base.DeferredSum)

    def forward(self, x, out_dtype, rows=None, packed=False, deferred=None):
        n = x.shape[0] if rows is None else rows.shape[0]
        if packed:
            out = ops.packed_rows(n, self.width, x.device)
        else:
            out = torch.empty((n, self.width), dtype=out_dtype, device=x.device)
        if deferred is not None and deferred.filled:
            if rows is None and self.width <= 8192:
                part, bias = deferred.part, deferred.bias
                deferred.part = deferred.bias = None
                return ops.layernorm_join(x, part, bias, self.weight, self.bias, self.eps, out)
            deferred.flush(x)
        return ops.layernorm(x, self.weight, self.bias, self.eps, out, rows)
