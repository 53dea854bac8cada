"""RMSNorm fused with the residual add in front of it.

``residual += delta`` in float32, then ``residual * rsqrt(mean(residual^2) + eps) * w``
(rapid_llm/kernels/ops/layernorm/skip_rmsnorm.py:41-47,:51-85).  The residual stream is
kept in float32 in every engine type; the reference rounds it to the activation type after
each add (:104-144), which this engine does not need to.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import NORMS, Norm, ParamSpec, Source
from .lazy import DeferredProduct


class RMSNorm(Norm):
    replayable = True
    fuses_products = True  # takes a DeferredProduct as delta, may return ScaledRows

    def __init__(self, size: int, eps: float, checkpoint_name: str, name: str = "norm") -> None:
        self.size = size
        self.eps = float(eps)
        self.checkpoint_name = checkpoint_name
        self.name = name
        self.weight: torch.Tensor | None = None

    def param_specs(self) -> list[ParamSpec]:
        return [
            ParamSpec(
                self.name + ".weight",
                (self.size,),
                "vector",
                (Source(self.checkpoint_name, self.size),),
                init="norm",
            )
        ]

    def bind(self, params, runtime) -> None:
        self.weight = params[self.name + ".weight"]
        self.dtype = runtime.dtype

    def forward(self, residual, delta, ctx, rows=None, scaled_ok=False):
        if isinstance(delta, DeferredProduct):
            if (
                scaled_ok and rows is None and delta.linear.out_features == self.size
                and self.dtype == torch.bfloat16 and delta.linear.bias is None and delta.linear.skinny(delta.x)
            ):
                # the producer's kernel adds into the residual and leaves what the consumer's
                # kernel needs to finish the norm: no kernel of this norm's own runs
                return delta.linear.add_to_residual(delta.x, residual, self.weight, self.eps)
            if (
                rows is None and delta.linear.out_features == self.size and self.dtype == torch.bfloat16
                and self.size % 4 == 0 and self.size <= 16 * 1024 and delta.linear.bias is None
                and delta.linear.midsize(delta.x)
            ):
                # the product arrives as float32 runs of K, which this norm's kernel adds
                out = torch.empty((residual.shape[0], self.size), dtype=self.dtype, device=residual.device)
                ops.add_rmsnorm_parts(residual, delta.linear.partial_sums(delta.x), self.weight, out, self.eps)
                return out
            delta = delta.materialize()
        n = residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.size), dtype=self.dtype, device=residual.device)
        ops.add_rmsnorm(residual, delta, self.weight, out, self.eps, rows)
        return out


NORMS.register("rmsnorm", RMSNorm)
