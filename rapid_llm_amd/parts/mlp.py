"""Dense SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))``.

Gate and up are one packed matrix ``[2I, H]`` with rows ``[gate | up]``
(rapid_llm/models/base.py:401-404, rapid_llm/modules/linear.py:157-172), so one product
feeds the activation kernel (rapid_llm/modules/mlp.py:67-68).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, ParamSpec, Source
from .lazy import ScaledRows
from .linear import Linear


class SwiGLU(FeedForward):
    replayable = True

    def __init__(
        self,
        hidden_size: int,
        intermediate_size: int,
        checkpoint_prefix: str,
        name: str = "ff",
        gate_name: str = "gate_proj.weight",
        up_name: str = "up_proj.weight",
        down_name: str = "down_proj.weight",
    ) -> None:
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.prefix = checkpoint_prefix
        self.name = name
        self.names = (gate_name, up_name, down_name)
        self.gate_up = Linear(hidden_size, 2 * intermediate_size)
        self.down = Linear(intermediate_size, hidden_size)

    def param_specs(self) -> list[ParamSpec]:
        h, i = self.hidden_size, self.intermediate_size
        g, u, d = (self.prefix + n for n in self.names)
        return [
            ParamSpec(self.name + ".gate_up", (2 * i, h), "matrix", (Source(g, i), Source(u, i))),
            ParamSpec(self.name + ".down", (h, i), "matrix", (Source(d, h),)),
        ]

    def bind(self, params, runtime) -> None:
        self.gate_up.bind(params[self.name + ".gate_up"])
        self.down.bind(params[self.name + ".down"])

    @property
    def accepts_scaled_rows(self) -> bool:
        return self.gate_up.takes_scaled_rows()

    def forward(self, x, ctx):
        w = self.gate_up.weight
        if w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16:
            # few rows: product and activation in one kernel
            act = ops.gemm_bf16_swiglu(x.rows, w, scaled=x) if isinstance(x, ScaledRows) else ops.gemm_bf16_swiglu(x, w)
            if act is not None:
                return self.down.deferred(act, ctx)
        gu = self.gate_up(x)
        act = torch.empty((x.shape[0], self.intermediate_size), dtype=gu.dtype, device=x.device)
        ops.swiglu(gu, act)
        return self.down.deferred(act, ctx)


FEED_FORWARDS.register("swiglu", SwiGLU)
