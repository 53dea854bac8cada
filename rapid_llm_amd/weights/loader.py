"""Weights by tensor name: safetensors -> the tensors a model's parts declared.

The model lists what it needs as :class:`~rapid_llm_amd.parts.base.ParamSpec` (name,
shape, role, checkpoint sources).  The loader streams the checkpoint one tensor at a
time (rapid_llm/executor/weight_utils.py:100-133), copies every source into its block of
rows, and checks coverage in both directions.  All problems of one load are reported
together in a single :class:`WeightsError`: tensors the model needs that the checkpoint
lacks, tensors the checkpoint has that nothing reads, and shape mismatches by name
(rapid_llm/models/weights.py:187-194,:217-239 report the same classes one at a time).

Storage types: in a float32 engine everything becomes float32.  In a bfloat16 engine
matrices stored in 16-bit are held as bfloat16, a matrix the checkpoint stores in 32-bit
stays 32-bit, per-channel vectors are float32 (exact for bfloat16 values) and integer
tables are int32.
"""

from __future__ import annotations

import re
from pathlib import Path
from typing import Iterable, Iterator, Sequence

import torch

from ..parts.base import ParamSpec

_FLOAT_TYPES = (torch.float32, torch.bfloat16, torch.float16, torch.float64)


class WeightsError(RuntimeError):
    """Checkpoint and model disagree.  ``missing``, ``unexpected`` and ``wrong_shape`` hold
    the names; the message lists them."""

    def __init__(self, where: str, missing, unexpected, wrong_shape, other=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.other = list(other)
        lines = [f"cannot load weights from {where}:"]

        def _section(title, items):
            if items:
                lines.append(f"  {title} ({len(items)}):")
                lines.extend(f"    {item}" for item in items)

        _section("missing tensors (the model needs them, the checkpoint has none)", self.missing)
        _section("unexpected tensors (in the checkpoint, read by nothing)", self.unexpected)
        _section("wrong shapes", self.wrong_shape)
        _section("other problems", self.other)
        super().__init__("\n".join(lines))


def checkpoint_files(model_dir: str | Path) -> list[Path]:
    """``*.safetensors`` under the folder, sorted (rapid_llm/executor/weight_utils.py:28-47)."""
    model_dir = Path(model_dir)
    files = sorted(model_dir.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(
            f"no *.safetensors file under {str(model_dir)!r}; this engine loads safetensors "
            "checkpoints (or pass load_format='random' to draw weights from a seed)"
        )
    return files


def iterate_checkpoint(model_dir: str | Path) -> Iterator[tuple[str, torch.Tensor]]:
    """Yield ``(name, cpu tensor)`` for every tensor of every shard, names sorted per shard."""
    from safetensors import safe_open

    for path in checkpoint_files(model_dir):
        with safe_open(str(path), framework="pt", device="cpu") as shard:
            for name in sorted(shard.keys()):
                yield name, shard.get_tensor(name)


def storage_dtype(role: str, stored: torch.dtype, engine_dtype: torch.dtype) -> torch.dtype:
    if role == "table":
        return torch.int32
    if role == "vector":
        return torch.float32
    if engine_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32  # a tensor stored in 32-bit stays so
    return torch.bfloat16


def _ignored(name: str, rules: Sequence) -> bool:
    for rule in rules:
        m = re.fullmatch(rule.pattern, name)
        if m is None:
            continue
        if rule.min_index is None or int(m.group(1)) >= rule.min_index:
            return True
    return False


def load_params(
    specs: Sequence[ParamSpec],
    tensors: Iterable[tuple[str, torch.Tensor]],
    *,
    engine_dtype: torch.dtype,
    device: torch.device | str,
    ignore_rules: Sequence = (),
    where: str = "checkpoint",
) -> dict[str, torch.Tensor]:
    """Fill every parameter from its sources; raise one error naming every disagreement."""
    by_source: dict[str, tuple[ParamSpec, int, int]] = {}
    other: list[str] = []
    for spec in specs:
        offset = 0
        for src in spec.sources:
            if src.name in by_source:
                other.append(f"checkpoint tensor {src.name!r} is claimed by two parameters")
            by_source[src.name] = (spec, offset, src.rows)
            offset += src.rows
        if spec.sources and offset != spec.shape[0]:
            other.append(
                f"parameter {spec.name!r}: its sources cover {offset} rows of {spec.shape[0]}"
            )

    out: dict[str, torch.Tensor] = {}
    seen: set[str] = set()
    unexpected: list[str] = []
    wrong: list[str] = []
    for name, tensor in tensors:
        hit = by_source.get(name)
        if hit is None:
            if not _ignored(name, ignore_rules):
                unexpected.append(f"{name} {tuple(tensor.shape)}")
            continue
        if name in seen:
            other.append(f"checkpoint tensor {name!r} appears twice")
            continue
        seen.add(name)
        spec, offset, rows = hit
        want = (rows, *spec.shape[1:])
        if tuple(tensor.shape) != want:
            wrong.append(
                f"{name}: checkpoint has {tuple(tensor.shape)}, parameter {spec.name!r} "
                f"expects {want}"
            )
            continue
        if spec.role == "table":
            if tensor.dtype in _FLOAT_TYPES:
                other.append(f"{name}: an integer table is stored as {tensor.dtype}")
                continue
        elif tensor.dtype not in _FLOAT_TYPES:
            other.append(f"{name}: stored as {tensor.dtype}, which this engine does not load")
            continue
        dest = out.get(spec.name)
        dtype = storage_dtype(spec.role, tensor.dtype, engine_dtype)
        if dest is None:
            dest = torch.empty(spec.shape, dtype=dtype, device=device)
            out[spec.name] = dest
        elif dest.dtype != dtype:
            # blocks of one fused matrix stored in different widths: keep the wider
            if dtype == torch.float32:
                dest = dest.to(torch.float32)
                out[spec.name] = dest
        dest[offset : offset + rows].copy_(tensor, non_blocking=False)

    missing: list[str] = []
    for spec in specs:
        absent = [s.name for s in spec.sources if s.name not in seen]
        if not absent:
            continue
        if len(absent) == len(spec.sources) and spec.fallback is not None:
            continue  # resolved below by sharing
        missing.extend(f"{n} (for parameter {spec.name!r})" for n in absent)
    if missing or unexpected or wrong or other:
        raise WeightsError(where, missing, unexpected, wrong, other)
    for spec in specs:
        if spec.name not in out and spec.fallback is not None:
            out[spec.name] = out[spec.fallback]  # one tensor, two names (tied projection)
    return out


def load_model_dir(
    model_dir: str | Path,
    specs: Sequence[ParamSpec],
    *,
    engine_dtype: torch.dtype,
    device: torch.device | str,
    ignore_rules: Sequence = (),
) -> dict[str, torch.Tensor]:
    return load_params(
        specs,
        iterate_checkpoint(model_dir),
        engine_dtype=engine_dtype,
        device=device,
        ignore_rules=ignore_rules,
        where=str(model_dir),
    )
