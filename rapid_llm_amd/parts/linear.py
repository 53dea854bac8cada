"""``y = x W^T (+ b)`` with ``W [out, in]`` as the checkpoint stores it.  This family has no
bias; a part of another architecture binds one, which is added by a kernel of its own after
the product (a product with a bias folds no norm into itself).

Which product runs is decided by the weight's storage type:

* float32 weight: the hand-written float32 FMA kernel (true 32-bit; the only product of
  the float32 engine).  A bfloat16 activation is widened first, so a matrix that the
  checkpoint stores in 32-bit is used at full precision in a bfloat16 engine too.
* bfloat16 weight: few rows (decode) go to the hand-written bandwidth-bound matrix-core
  kernel; many rows go to the library product, as in the reference, whose dense products
  are ``F.linear`` (rapid_llm/kernels/ops/gemm/linear.py:17-40).  In between (17 to 192 rows) a
  narrow matrix whose result a norm adds to the residual may hand that norm float32 runs of
  K instead (``partial_sums``).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .lazy import DeferredProduct, ScaledRows


class Linear:
    def __init__(self, in_features: int, out_features: int) -> None:
        self.in_features = in_features
        self.out_features = out_features
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None

    def bind(self, weight: torch.Tensor, bias: torch.Tensor | None = None) -> None:
        if tuple(weight.shape) != (self.out_features, self.in_features):
            raise ValueError(
                f"linear weight must be {(self.out_features, self.in_features)}, is {tuple(weight.shape)}"
            )
        if bias is not None and (tuple(bias.shape) != (self.out_features,) or bias.dtype != torch.float32):
            raise ValueError(f"linear bias must be float32 of shape {(self.out_features,)}, is {bias.dtype} {tuple(bias.shape)}")
        self.weight = weight
        self.bias = bias

    # ---- folding a neighbouring norm into the product (decode steps, bfloat16) ----------
    def skinny(self, x) -> bool:
        """Whether ``x`` runs through the hand-written few-row kernel, which has the epilogues."""
        return (
            self.weight.dtype == torch.bfloat16 and x.dtype == torch.bfloat16
            and x.shape[0] <= ops.SKINNY_MAX_ROWS and self.in_features % 8 == 0
        )

    def folds(self, x) -> bool:
        """Whether this product may absorb the residual add and norm that follow it: one of the
        two kernels with that epilogue runs it, and no bias comes between."""
        return self.bias is None and (self.skinny(x) or self.midsize(x))

    def takes_scaled_rows(self) -> bool:
        """Whether this product can finish a norm whose rows arrive unscaled (whatever the
        few rows of a step are): only the few-row kernel has that epilogue."""
        return self.weight is not None and self.weight.dtype == torch.bfloat16 and self.in_features % 8 == 0

    def midsize(self, x) -> bool:
        """Whether ``x`` (more rows than the few-row kernel takes) may run as float32 runs of K
        that a norm adds (narrow matrices only: the wide ones are faster in the library)."""
        return (
            self.weight.dtype == torch.bfloat16 and x.dtype == torch.bfloat16
            and ops.SKINNY_MAX_ROWS < x.shape[0] <= ops.MID_MAX_ROWS
            and ops.mid_runs(self.out_features, self.in_features) > 0
        )

    def partial_sums(self, x: torch.Tensor) -> torch.Tensor:
        """``[runs, M, out]`` float32 whose sum over the runs is ``x W^T``."""
        return ops.gemm_bf16_parts(x, self.weight)

    def deferred(self, x: torch.Tensor, ctx=None):
        """The product, or a :class:`DeferredProduct` of it where one of this product's kernels
        could fold a neighbouring norm into itself (bfloat16, up to 16 rows, or 17 to 192 rows of a
        narrow matrix).  Whoever receives it and has no use for that simply materialises it."""
        if isinstance(x, torch.Tensor) and self.folds(x):
            return DeferredProduct(self, x)
        return self(x)

    def add_to_residual(
        self, x: torch.Tensor, residual: torch.Tensor, norm_weight: torch.Tensor, eps: float
    ) -> ScaledRows:
        """``residual += x W^T`` in place; returns the new rows times ``norm_weight`` and the
        pieces of their sums of squares."""
        rows, partial = ops.gemm_bf16_residual(x, self.weight, residual, norm_weight)
        return ScaledRows(rows, partial, self.out_features, eps)

    def __call__(self, x, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        w = self.weight
        if isinstance(x, ScaledRows):
            if not self.skinny(x):
                raise ValueError("scaled rows reached a product that cannot apply their factor")
            y = ops.gemm_bf16(x.rows, w, out_dtype or x.dtype, scaled=x)
            if self.bias is not None:
                ops.add_bias(y, self.bias)
            return y
        rows = x.shape[0]
        out_dtype = out_dtype or x.dtype
        if w.dtype == torch.float32:
            if x.dtype != torch.float32:
                wide = torch.empty(x.shape, dtype=torch.float32, device=x.device)
                ops.cast(x, wide)
                x = wide
            y = torch.empty((rows, self.out_features), dtype=torch.float32, device=x.device)
            ops.gemm_f32(x, w, y)
        else:
            y = ops.gemm_bf16(x, w, out_dtype)
        if y.dtype != out_dtype:
            narrow = torch.empty(y.shape, dtype=out_dtype, device=y.device)
            ops.cast(y, narrow)
            y = narrow
        if self.bias is not None:
            ops.add_bias(y, self.bias)
        return y
