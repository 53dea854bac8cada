"""Random weights from a configuration and a seed.

``write_random_model`` writes a model folder (``config.json`` + ``model.safetensors``)
that loads like any checkpoint; ``random_params`` fills the model's parameters on the
device directly (the benchmark shapes are tens of gigabytes and never touch the disk).

The reference has random weights only in its single-layer harness: one generator, norm
weights 1, everything else N(0, 0.02) drawn in float32
(rapid_llm/tools/harness/single_layer.py:33-37,:478-504).  Here the whole model is drawn,
checkpoint tensor by checkpoint tensor in the order the model lists them, from one CPU
generator; norm weights are ``1 + N(0, norm_std)``.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping, Sequence

import torch

from ..parts.base import ParamSpec

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def _draw(shape, init: str, gen: torch.Generator, std: float, norm_std: float, device="cpu"):
    if init == "norm":
        t = torch.ones(shape, dtype=torch.float32, device=device)
        if norm_std:
            t += torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * norm_std
        return t
    if init == "zeros":
        return torch.zeros(shape, dtype=torch.float32, device=device)
    if init == "normal":
        return torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * std
    raise ValueError(f"unknown init {init!r}")


def random_checkpoint_tensors(
    specs: Sequence[ParamSpec],
    seed: int,
    *,
    dtype: str = "bfloat16",
    std: float = 0.02,
    norm_std: float = 0.1,
) -> dict[str, torch.Tensor]:
    """Checkpoint-named tensors for every source of every parameter (CPU)."""
    gen = torch.Generator().manual_seed(int(seed))
    out: dict[str, torch.Tensor] = {}
    for spec in specs:
        if spec.fallback is not None:
            continue  # shared with another parameter: the checkpoint ships none
        for src in spec.sources:
            shape = (src.rows, *spec.shape[1:])
            t = _draw(shape, spec.init, gen, std, norm_std)
            out[src.name] = t.to(_STORE[dtype]) if spec.role != "table" else t.to(torch.int32)
    return out


def write_random_model(
    config: Any,
    seed: int,
    out_dir: str | Path,
    *,
    dtype: str | None = None,
    std: float = 0.02,
    norm_std: float = 0.1,
) -> Path:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (a typed configuration
    or a ``config.json`` body) with weights drawn from ``seed``."""
    from safetensors.torch import save_file

    from ..config.registry import config_from_dict
    from ..models.causal_lm import model_param_specs

    body: Mapping[str, Any] = config if isinstance(config, Mapping) else config.to_dict()
    entry, cfg = config_from_dict(body)
    body = dict(cfg.to_dict())
    if dtype is not None:
        body["torch_dtype"] = dtype
    store = body.get("torch_dtype", "bfloat16")
    spec = entry.build_spec(cfg)
    tensors = random_checkpoint_tensors(
        model_param_specs(spec), seed, dtype=store, std=std, norm_std=norm_std
    )
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    (out_dir / "config.json").write_text(json.dumps(body, indent=2) + "\n")
    save_file(tensors, str(out_dir / "model.safetensors"))
    return out_dir


def random_params(
    specs: Sequence[ParamSpec],
    seed: int,
    *,
    engine_dtype: torch.dtype,
    device: torch.device | str,
    std: float = 0.02,
    norm_std: float = 0.0,
) -> dict[str, torch.Tensor]:
    """Parameters drawn on the device, without a checkpoint (benchmark shapes)."""
    gen = torch.Generator(device=device).manual_seed(int(seed))
    out: dict[str, torch.Tensor] = {}
    for spec in specs:
        if spec.fallback is not None:
            continue
        if spec.role == "vector":
            out[spec.name] = _draw(spec.shape, spec.init, gen, std, norm_std, device)
        elif spec.role == "table":
            out[spec.name] = torch.zeros(spec.shape, dtype=torch.int32, device=device)
        else:
            t = torch.empty(spec.shape, dtype=engine_dtype, device=device)
            t.normal_(0.0, std, generator=gen)
            out[spec.name] = t
    for spec in specs:
        if spec.fallback is not None:
            out[spec.name] = out[spec.fallback]
    return out
