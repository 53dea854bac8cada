"""Token selection on the device: one kernel call per step for all rows of the batch.

Rows that are all greedy and unpenalised take the arg-max kernel; anything else takes the
general kernel (repetition penalty, temperature, nucleus, seeded draw), which handles
greedy and stochastic rows of one batch alike, as the reference merges them per row
(rapid_llm/engine/sampler.py:691-696).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence

import numpy as np
import torch

from ..kernels import ops


@dataclass
class RowSampling:
    """What the kernel needs to pick one row's token."""

    temperature: float = 0.0
    top_p: float = 1.0
    repetition_penalty: float = 1.0
    seed: int = 0
    counter: int = 0  # tokens the request has generated so far
    generated: Sequence[int] = field(default_factory=tuple)  # read when the penalty is on


class Sampler:
    def __init__(self, device: torch.device | str = "cuda") -> None:
        self.device = torch.device(device)

    def sample(
        self, logits: torch.Tensor, rows: Sequence[RowSampling], want_logprobs: bool = False
    ) -> tuple[torch.Tensor, torch.Tensor | None]:
        """``logits [R, vocab]`` float32 -> chosen ids ``[R]`` int32 (on the device) and,
        if asked, the chosen tokens' log-probabilities ``[R]`` float32."""
        n = logits.shape[0]
        if n != len(rows):
            raise ValueError(f"{n} rows of logits for {len(rows)} sampling rows")
        out = torch.empty(n, dtype=torch.int32, device=self.device)
        if n == 0:
            return out, (torch.empty(0, dtype=torch.float32, device=self.device) if want_logprobs else None)
        plain = all(r.temperature == 0.0 and r.repetition_penalty == 1.0 for r in rows)
        if plain and not want_logprobs:
            ops.argmax(logits, out)
            return out, None
        any_penalty = any(r.repetition_penalty != 1.0 and len(r.generated) > 0 for r in rows)
        params = np.zeros((n, 8), dtype=np.int32)
        fl = params.view(np.float32)
        history: list[int] = []
        for i, r in enumerate(rows):
            fl[i, 0] = r.temperature
            fl[i, 1] = r.top_p
            fl[i, 2] = r.repetition_penalty
            seed = int(r.seed) & ((1 << 64) - 1)
            params[i, 3] = np.uint32(seed & 0xFFFFFFFF).astype(np.int32)
            params[i, 4] = np.uint32(seed >> 32).astype(np.int32)
            params[i, 5] = np.uint32(r.counter & 0xFFFFFFFF).astype(np.int32)
            params[i, 6] = len(history)
            if r.repetition_penalty != 1.0:
                history.extend(int(t) for t in r.generated)
            params[i, 7] = len(history)
        packed = np.concatenate([params.reshape(-1), np.asarray(history, dtype=np.int32)])
        dev = torch.from_numpy(packed).to(self.device)
        logprob = torch.empty(n, dtype=torch.float32, device=self.device) if want_logprobs else None
        ops.sample(
            logits, dev[: 8 * n], dev[8 * n :] if history else None, out, logprob, any_penalty
        )
        return out, logprob
