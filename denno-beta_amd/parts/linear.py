"""Linear: a weight held [out, in] with an optional 32-bit bias, and the call that picks the
product for its dtype.  A weight that a checkpoint stores [in, out] (Conv1D,
crates/denno-engine/src/quant.rs:951-953) is transposed once at load (ParamSpec.transpose).
A bfloat16 weight on the GPU is packed once at bind for the matrix cores (ops.PackedMatrix);
the rows it came from are not kept, unless another part holds them (a tied table)."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from ..weights.spec import ParamSpec
from .base import LazyNorm


class Linear:
    def __init__(self, in_features: int, out_features: int, weight_name: str, bias_name: Optional[str],
                 stored_in_out: bool = False, init_std: float = 0.02, weight_sources=None, bias_sources=None):
        """weight_sources, bias_sources: ((file name, output columns), ...): the checkpoint stores the weight
        (the bias) as several tensors, one per run of output columns (q, k and v of a fused projection; gate
        and up); they are joined once, at load, and `weight_name` / `bias_name` then name only what is held."""
        self.in_features, self.out_features = in_features, out_features
        self.weight_name, self.bias_name = weight_name, bias_name
        self.stored_in_out = stored_in_out
        self.init_std = init_std
        self.weight_sources = tuple((n, int(c)) for n, c in weight_sources) if weight_sources else None
        self.bias_sources = tuple((n, int(c)) for n, c in bias_sources) if bias_sources else None
        if self.bias_sources and not bias_name:
            raise ValueError("Linear: bias_sources need a bias_name to hold them under")
        self.weight = None
        self.bias = None
        self._folded = {}      # id(norm) -> (c1, c2, eps): see fold_norm

    def param_specs(self):
        shape = (self.in_features, self.out_features) if self.stored_in_out else (self.out_features, self.in_features)
        # (the output columns are the stored layout's first dimension, or its second where it is [in, out])
        specs = [ParamSpec(self.weight_name, shape, "matrix", ("normal", 0.0, self.init_std),
                           transpose=self.stored_in_out, sources=self.weight_sources,
                           concat_dim=1 if self.stored_in_out else 0)]
        if self.bias_name:
            specs.append(ParamSpec(self.bias_name, (self.out_features,), "vector", ("normal", 0.0, 0.01),
                                   sources=self.bias_sources))
        return specs

    def bind(self, tensors):
        w = tensors[self.weight_name]
        if w.dtype == torch.bfloat16 and w.is_cuda and w.shape[1] % 8 == 0:
            w = ops.pack_matrix(w)
        self.weight = w
        self.bias = tensors[self.bias_name] if self.bias_name else None

    def few_rows(self, n_rows: int) -> bool:
        """Whether a call with n_rows rows runs the few-rows product, which reads and writes packed rows."""
        return isinstance(self.weight, ops.PackedMatrix) and n_rows <= ops.PACKED_ROWS_MAX

    def packed_input(self, n_rows: int) -> bool:
        """Whether the rows for a call with n_rows rows should be made as packed rows
        (ops.packed_rows): whoever makes them asks here.  From 17 to 256 rows: a wave of the few-rows
        product then reads 1 KB in one piece where rows of the ordinary layout cost it 16 cache
        lines per 16 lanes (up to 16 rows its kernel loads along rows and turns them round in LDS;
        beyond 256 the many-rows kernels read rows)."""
        return self.few_rows(n_rows) and n_rows >= ops.PACKED_ROWS_MIN and self.in_features % 32 == 0

    def fold_norm(self, norm):
        """Makes ready to run `norm` (the norm that stands before this product) inside the product's
        own kernel: ops.norm_folded, once."""
        f = getattr(norm, "fused_params", None)
        if f is None or not (ops.norm_stream_takes(1, self.in_features, self.weight)
                             or ops.norm_stream_takes(17, self.in_features, self.weight)):
            return
        # kinds: "layernorm" ((x - mean) / sqrt(var + eps) * gamma + beta) and "rmsnorm" (x / sqrt(mean(x^2) + eps)
        # * gamma, beta None); a norm of another kind runs as its own kernel
        kind, gamma, beta, eps = f()
        if kind == "layernorm":
            self._folded[id(norm)] = (*ops.norm_folded(self.weight.rows(), self.bias, gamma, beta), eps, False)
        elif kind == "rmsnorm" and beta is None:
            self._folded[id(norm)] = (*ops.norm_folded(self.weight.rows(), self.bias, gamma, None, no_mean=True), eps, True)

    def takes_lazy_norm(self, n_rows: int, norm) -> bool:
        """Whether a call with n_rows rows can run `norm` in its own kernel (fold_norm has been called)."""
        return id(norm) in self._folded and ops.norm_stream_takes(n_rows, self.in_features, self.weight)

    def writes_norm_stats(self, n_rows: int) -> bool:
        """Whether a call with n_rows rows that adds into the residual stream can leave what the norm after it needs."""
        return ops.norm_stream_takes(n_rows, self.out_features, self.weight) and self.in_features % 8 == 0

    def defers(self, n_rows: int) -> bool:
        """Whether a call with n_rows rows that adds into the residual stream can leave its sum for the next norm's kernel."""
        return ops.linear_deferred_shares(n_rows, self.weight) > 0

    def _fusable(self, a, out_dtype):
        """(c1, c2, eps, no_mean) if `a` is a LazyNorm that this call can run in its own kernel."""
        if ((out_dtype or a.dtype) == torch.bfloat16 and a.stream is not None and a.stream.written
                and a.stream.norm is a.norm and self.takes_lazy_norm(a.shape[0], a.norm)):
            return self._folded[id(a.norm)]
        return None

    def __call__(self, a, out_dtype=None, epilogue="none", residual=None, packed_out=False, stats=None, deferred=None):
        """epilogue(a @ W^T + b) as a new [M, out] tensor of out_dtype (as packed rows if
        packed_out, for a Linear whose packed_input said so), or added into `residual` (32-bit) in
        place (or, with `deferred`, an empty parts.base.DeferredSum, left there for the next norm's kernel to add,
        where `defers` says so).  An input in another precision than the weight is converted to the weight's (exact
        from bfloat16 to 32-bit)."""
        if isinstance(a, LazyNorm):
            f = self._fusable(a, out_dtype) if residual is None and not (packed_out and a.shape[0] <= 16) else None
            if f is not None:
                out = (ops.packed_rows(a.shape[0], self.out_features, a.device) if packed_out else
                       torch.empty((a.shape[0], self.out_features), dtype=torch.bfloat16, device=a.device))
                return ops.linear_norm_in(a.stream.copy, a.stream.stats, f[0], f[1], f[2], self.weight, out, epilogue=epilogue,
                                          no_mean=f[3])
            a = a.rows(packed=self.packed_input(a.shape[0]))
        if a.dtype != self.weight.dtype:
            a = ops.cast(a.contiguous(), torch.empty(a.shape, dtype=self.weight.dtype, device=a.device))
        if residual is not None:
            if deferred is not None and a.dtype == torch.bfloat16 and self.defers(a.shape[0]):
                deferred.fill(ops.linear_deferred(a, self.weight), self.bias)       # (the stream itself stays as it is)
                return residual
            if stats is not None and a.dtype == torch.bfloat16 and self.writes_norm_stats(a.shape[0]):
                stats.written = True
                return ops.linear_norm_out(a, self.weight, self.bias, residual, stats.norm.fused_params()[1],
                                           stats.copy, stats.stats)
            return ops.linear(a, self.weight, self.bias, residual=residual)
        if packed_out:
            out = ops.packed_rows(a.shape[0], self.out_features, a.device)
        else:
            out = torch.empty((a.shape[0], self.out_features), dtype=out_dtype or a.dtype, device=a.device)
        return ops.linear(a, self.weight, self.bias, out=out, epilogue=epilogue)

    def project_qkv(self, a, out_dtype, slot_map, k_pool, v_pool, q_width):
        """The fused projection: the key and value columns go to the cache's pages, the queries
        [M, q_width] come back (where one kernel does both, the other columns are stored nowhere else)."""
        if isinstance(a, LazyNorm):
            f = self._fusable(a, out_dtype)
            if f is not None:
                out = torch.empty((a.shape[0], q_width), dtype=torch.bfloat16, device=a.device)
                return ops.linear_norm_in(a.stream.copy, a.stream.stats, f[0], f[1], f[2], self.weight, out,
                                          kv=(slot_map, k_pool, v_pool, q_width), no_mean=f[3])
            a = a.rows(packed=self.packed_input(a.shape[0]))
        if a.dtype != self.weight.dtype:
            a = ops.cast(a.contiguous(), torch.empty(a.shape, dtype=self.weight.dtype, device=a.device))
        fused = isinstance(self.weight, ops.PackedMatrix) and out_dtype == torch.bfloat16
        out = torch.empty((a.shape[0], q_width if fused else self.out_features), dtype=out_dtype, device=a.device)
        return ops.linear_qkv(a, self.weight, self.bias, out, slot_map, k_pool, v_pool, q_width)
