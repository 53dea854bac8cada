"""How close a bfloat16 engine has to come to the plain implementation, and the models on
which a lost key shows.

The oracle is the plain implementation in float32 on the weights as the bfloat16 checkpoint
stores them, so what remains is the engine's own rounding of activations and cache.  Two
figures are taken per comparison, both relative to the spread of the logits (their standard
deviation over the compared block):

* ``row``: the worst row's root-mean-square error.  Rounding noise averages out over a
  row, a lost or stale key moves the whole row: this is the figure that tells them apart.
* ``peak``: the worst single element, against a single corrupted logit.  The largest of n
  rounding errors grows with n (a row of 151,936 logits against one of 256), so its bound is
  the row bound times ``sqrt(2 ln n)``, what the largest of n normal errors of that size reaches.

The row bound is twice the worst figure seen on an MI355X over every tiny configuration and
every way of cutting the requests, and 1.7 times the worst at the benchmark's widths
(``RAPID_LLM_PARITY_LOG=file`` makes a run append what it saw; in absolute terms the worst
element was off by 0.007 where logits spread by 0.2, and by 0.08 where they spread by 1.28).  Rounding
the plain implementation's own activations to bfloat16 wherever an engine stores them moves its
logits by about as much, and no closer to an engine's: the roundings are not the same ones, so
that result is no tighter oracle, only a measure of what rounding alone does.
``tests/test_parity_bound.py`` shows on the CPU what the bounds reject: a key that later
queries have lost, every query's own key, the own key of the last 32 tokens in one layer, a
run of 128 keys at the end of a long context, a window one key too long or too short, one
logit moved by a tenth of the spread.  What they cannot reject is one key among hundreds lost
by one late row (it moves that row by less than rounding does): that is the kernel tests'
part, with keys made to stand out.
"""

from __future__ import annotations

import json
import math
import os
from pathlib import Path

import torch

BF16_ROW = 0.02  # worst row's rms error / spread of the logits (worst seen: 0.0102 tiny, 0.0121 at real widths)


def peak_bound(elements: int) -> float:
    """Worst element's error / spread of the logits among ``elements`` compared ones (worst seen:
    0.034 of 0.091 among 25,600, 0.062 of 0.113 among 7 million)."""
    return BF16_ROW * math.sqrt(2.0 * math.log(max(elements, 2)))


def errors(got: torch.Tensor, want: torch.Tensor) -> tuple[float, float, int]:
    """(row, peak, worst row's index) of ``got`` against ``want``, both ``[rows, vocab]``."""
    diff = got.double() - want.double()
    spread = float(want.double().std())
    rows = diff.square().mean(dim=1).sqrt() / spread
    peak = float(diff.abs().max()) / spread
    worst = int(rows.argmax())
    return float(rows[worst]), peak, worst


def record(label: str, row: float, peak: float) -> None:
    print(f"parity {label}: row {row:.4f} peak {peak:.4f} of the logits' spread")
    path = os.environ.get("RAPID_LLM_PARITY_LOG")
    if path:
        with open(path, "a") as f:
            f.write(json.dumps({"label": label, "row": round(row, 5), "peak": round(peak, 5)}) + "\n")


def assert_bf16_close(got: torch.Tensor, want: torch.Tensor, label: str) -> None:
    assert got.shape == want.shape, (label, tuple(got.shape), tuple(want.shape))
    assert torch.isfinite(got).all(), f"{label}: non-finite logits"
    row, peak, worst = errors(got, want)
    record(label, row, peak)
    peak_limit = peak_bound(got.numel())
    if row > BF16_ROW or peak > peak_limit:
        diff = (got.double() - want.double()).square().mean(dim=1).sqrt() / float(want.double().std())
        beyond = torch.nonzero(diff > BF16_ROW)
        first = int(beyond[0]) if beyond.numel() else worst
        raise AssertionError(
            f"{label}: bfloat16 logits are off by row {row:.4f} (bound {BF16_ROW}) / peak {peak:.4f} "
            f"(bound {peak_limit:.4f}) of their spread; worst row {worst}, first row beyond the bound {first}"
        )


def assert_near_choice(logits_row: torch.Tensor, token: int, label: str) -> None:
    """A greedy bfloat16 engine may pick another of several nearly equal maxima, never a token
    whose plain logit is further below the plain maximum than two logits can be off together."""
    gap = float(logits_row.max() - logits_row[token])
    bound = 2 * peak_bound(logits_row.numel()) * float(logits_row.double().std())
    assert gap <= bound, f"{label}: the chosen token {token} lies {gap:.4f} below the plain maximum (bound {bound:.4f})"


def to_bf16(x: torch.Tensor) -> torch.Tensor:
    """The rounding a bfloat16 engine applies wherever it stores an activation."""
    return x.bfloat16().to(x.dtype)


def sharpen(model_dir: Path, gain: float = 2.5) -> Path:
    """Scale every layer's q and k head-norm weights by ``gain``: scores grow by ``gain`` squared,
    a few keys then carry most of each query's weight, and losing one of them moves that query's
    output by much more than rounding does.  Both the engine and the plain implementation read
    the folder afterwards."""
    from safetensors.torch import load_file, save_file

    path = str(Path(model_dir) / "model.safetensors")
    tensors = load_file(path)
    for name in list(tensors):
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            tensors[name] = (tensors[name].float() * gain).to(tensors[name].dtype)
    save_file(tensors, path)
    return Path(model_dir)
