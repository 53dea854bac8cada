"""What every part is told about the engine it runs in."""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Runtime:
    device: torch.device
    dtype: torch.dtype  # compute type of activations and cache: bfloat16 or float32
    max_seq_len: int  # longest sequence a request may reach (sizes position tables)
    page_size: int
