"""Grouped-query attention over the paged cache.

Per step: fused QKV projection (rapid_llm/models/base.py:121-132), per-head RMSNorm of q
and k over head_dim before the rotation (:134-137), rotation (:139-140), write of this
step's keys and values into their pages (rapid_llm/modules/attention.py:126-138), attention
of every query over its request's cached keys up to its own position (:157-240), output
projection (base.py:164-165).  The norm, the rotation and the cache write are one kernel.
How the rotation is applied is the position part's to say (its tables' width: how many of a
head's channels rotate; its ``pairing``: which of them form a pair); the kernels here take
every such case, the fastest ones the half-split rotation of the whole head.

Keys and values are always read back from the pages, also for the tokens of the current
step, so that one code path serves whole prompts, portions and single decoded tokens
(the reference switches kernels by phase, attention.py:179-240).  ``window`` > 0 limits a
query at position p to keys ``[p - window + 1, p]`` (rapid_llm/engine/kv_cache_spec.py:203-222).
"""

from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Mixer, ParamSpec, Source
from .linear import Linear


class GQAAttention(Mixer):
    replayable = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        checkpoint_prefix: str,
        qk_norm_eps: float | None = None,
        window: int = 0,
        position=None,
        softmax_scale: float | None = None,
        name: str = "mixer",
        q_name: str = "q_proj.weight",
        k_name: str = "k_proj.weight",
        v_name: str = "v_proj.weight",
        o_name: str = "o_proj.weight",
        q_norm_name: str = "q_norm.weight",
        k_norm_name: str = "k_norm.weight",
        qkv_bias: bool = False,
        o_bias: bool = False,
    ) -> None:
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not divisible by {num_kv_heads} kv heads")
        if head_dim % 8 or not 8 <= head_dim <= 256:
            raise ValueError(f"attention kernels take head sizes in steps of 8 up to 256, got {head_dim}")
        self.hidden_size = hidden_size
        self.nq, self.nkv, self.d = num_heads, num_kv_heads, head_dim
        self.prefix = checkpoint_prefix
        self.qk_norm_eps = qk_norm_eps
        self.window = int(window)
        self.position = position
        # what the position part says about its rotation must be something the kernels can do
        rotary_dim = int(getattr(position, "rotary_dim", 0) or 0)
        pairing = getattr(position, "pairing", "half_split")
        if rotary_dim % 2 or rotary_dim > head_dim:
            raise ValueError(f"the position encoding rotates {rotary_dim} channels of heads of {head_dim}")
        if pairing not in ops.ROTARY_PAIRINGS:
            raise ValueError(
                f"the attention kernels rotate pairs as {sorted(ops.ROTARY_PAIRINGS)}, not as {pairing!r}"
            )
        self.scale = float(softmax_scale) if softmax_scale is not None else 1.0 / math.sqrt(head_dim)
        self.name = name
        self.names = dict(q=q_name, k=k_name, v=v_name, o=o_name, qn=q_norm_name, kn=k_norm_name)
        self.qkv = Linear(hidden_size, (num_heads + 2 * num_kv_heads) * head_dim)
        self.o = Linear(num_heads * head_dim, hidden_size)
        self.q_norm_w = self.k_norm_w = None
        # Qwen3 has neither (rapid_llm/models/qwen3.py:16-18: qkv_bias=False); architectures of the
        # same skeleton do (rapid_llm/models/base.py:121-132 passes bias=qkv_bias), under the
        # projections' names with ".bias" in place of ".weight"
        self.qkv_bias, self.o_bias = bool(qkv_bias), bool(o_bias)

    # ---- tensors ---------------------------------------------------------------
    def param_specs(self) -> list[ParamSpec]:
        p, n = self.prefix, self.names
        q_rows, kv_rows = self.nq * self.d, self.nkv * self.d
        specs = [
            ParamSpec(
                self.name + ".qkv",
                (q_rows + 2 * kv_rows, self.hidden_size),
                "matrix",
                (Source(p + n["q"], q_rows), Source(p + n["k"], kv_rows), Source(p + n["v"], kv_rows)),
            ),
            ParamSpec(self.name + ".o", (self.hidden_size, q_rows), "matrix", (Source(p + n["o"], self.hidden_size),)),
        ]
        if self.qk_norm_eps is not None:
            specs += [
                ParamSpec(self.name + ".q_norm", (self.d,), "vector", (Source(p + n["qn"], self.d),), init="norm"),
                ParamSpec(self.name + ".k_norm", (self.d,), "vector", (Source(p + n["kn"], self.d),), init="norm"),
            ]

        def bias_of(weight_name: str) -> str:
            return weight_name[: -len("weight")] + "bias" if weight_name.endswith("weight") else weight_name + ".bias"

        if self.qkv_bias:
            specs.append(ParamSpec(
                self.name + ".qkv_bias", (q_rows + 2 * kv_rows,), "vector",
                (Source(p + bias_of(n["q"]), q_rows), Source(p + bias_of(n["k"]), kv_rows),
                 Source(p + bias_of(n["v"]), kv_rows)),
            ))
        if self.o_bias:
            specs.append(ParamSpec(
                self.name + ".o_bias", (self.hidden_size,), "vector", (Source(p + bias_of(n["o"]), self.hidden_size),)
            ))
        return specs

    def bind(self, params, runtime) -> None:
        self.qkv.bind(params[self.name + ".qkv"], params[self.name + ".qkv_bias"] if self.qkv_bias else None)
        self.o.bind(params[self.name + ".o"], params[self.name + ".o_bias"] if self.o_bias else None)
        if self.qk_norm_eps is not None:
            self.q_norm_w = params[self.name + ".q_norm"]
            self.k_norm_w = params[self.name + ".k_norm"]
        self.runtime = runtime

    # ---- cache -----------------------------------------------------------------
    def cache_need(self) -> CacheNeed:
        return CacheNeed.keys_and_values(self.nkv, self.d, window=self.window)

    def recorded_step_bytes(self, rows: int, context_bound: int, page_size: int) -> int:
        return ops.decode_scratch_bytes(rows, self.nq, self.nkv, self.d, context_bound, page_size, self.window)

    # ---- step ------------------------------------------------------------------
    @property
    def accepts_scaled_rows(self) -> bool:
        return self.qkv.takes_scaled_rows()

    def forward(self, x, ctx, cache):
        tokens = x.shape[0]
        qkv = self.qkv(x)
        table = ctx.block_tables[cache.group_id]
        pos_enc = self.position
        cos = pos_enc.cos if pos_enc is not None else None
        sin = pos_enc.sin if pos_enc is not None else None
        eps = self.qk_norm_eps if self.qk_norm_eps is not None else 0.0
        out = torch.empty((tokens, self.nq * self.d), dtype=qkv.dtype, device=x.device)
        rotary_half = cos.shape[1] if cos is not None else 0
        pairing = getattr(pos_enc, "pairing", "half_split") if cos is not None else "half_split"
        if ops.decode_attention_fusable(ctx, qkv.dtype, self.nq // self.nkv, self.d, rotary_half, pairing):
            # a step of single tokens: norm, rotation, cache write and attention in one kernel
            ops.decode_attention_fused(
                qkv, cache.k, cache.v, out, ctx, table, cache.page_size, self.nq, self.nkv, self.d,
                self.window, self.scale, self.q_norm_w, self.k_norm_w, cos, sin, eps, cache.owns_pages,
            )
            return self.o.deferred(out, ctx)
        # where the attention kernels can finish the query heads as they read them, only the keys
        # and values are prepared here, and the queries are never written out
        in_kernel = ops.attention_prepares_queries(qkv.dtype, self.d, rotary_half, pairing)
        q = None if in_kernel else torch.empty((tokens, self.nq * self.d), dtype=qkv.dtype, device=x.device)
        ops.qknorm_rope_kvwrite(
            qkv, q,
            cache.k if cache.owns_pages else None,
            cache.v if cache.owns_pages else None,
            self.q_norm_w, self.k_norm_w, cos, sin,
            ctx.positions, ctx.token_slot, table, cache.page_size,
            self.nq, self.nkv, self.d, eps, ctx.max_position, pairing,
        )
        ops.paged_attention(
            qkv if in_kernel else q, cache.k, cache.v, out, ctx, table, cache.page_size,
            self.nq, self.nkv, self.d, self.window, self.scale,
            prepare=(self.q_norm_w, cos, sin, eps) if in_kernel else None,
        )
        return self.o.deferred(out, ctx)


MIXERS.register("gqa_attention", GQAAttention)
