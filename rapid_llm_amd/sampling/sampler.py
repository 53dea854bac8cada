"""Token selection on the device: one kernel call per step for all rows of the batch.

Rows that are all greedy and unpenalised take the arg-max kernel; anything else takes the
general kernel (repetition penalty, temperature, nucleus, seeded draw), which handles
greedy and stochastic rows of one batch alike, as the reference merges them per row
(rapid_llm/engine/sampler.py:691-696).  Log-probability records come from a kernel of their
own, run only for the rows that ask for them.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence

import numpy as np
import torch

from ..kernels import ops
from ..kernels.upload import upload, upload_ints
from .logprobs import PositionLogprobs


@dataclass
class RowSampling:
    """What the kernel needs to pick one row's token."""

    temperature: float = 0.0
    top_p: float = 1.0
    repetition_penalty: float = 1.0
    seed: int = 0
    counter: int = 0  # tokens the request has generated so far
    # read when the penalty is on; -(r + 1) names what sampling row r of the step before
    # chose, for a token the host has not read back yet
    generated: Sequence[int] = field(default_factory=tuple)


def _pack_rows(rows: Sequence[RowSampling], fed_rows: int = 0) -> tuple[np.ndarray, int, bool, bool]:
    """The kernels' per-row parameter words followed by the rows' generated tokens:
    ``(packed int32, words of parameters, whether any row is penalised, whether a history
    names a row of the step before)``; ``fed_rows`` is how many such rows there are."""
    n = len(rows)
    params = np.zeros((n, 8), dtype=np.int32)
    fl = params.view(np.float32)
    un = params.view(np.uint32)
    history: list[int] = []
    any_penalty = False
    for i, r in enumerate(rows):
        fl[i, 0] = r.temperature
        fl[i, 1] = r.top_p
        fl[i, 2] = r.repetition_penalty
        seed = int(r.seed) & ((1 << 64) - 1)
        un[i, 3] = seed & 0xFFFFFFFF
        un[i, 4] = seed >> 32
        un[i, 5] = r.counter & 0xFFFFFFFF
        params[i, 6] = len(history)
        if r.repetition_penalty != 1.0 and len(r.generated) > 0:
            history.extend(int(t) for t in r.generated)
            any_penalty = True
        params[i, 7] = len(history)
    tokens = np.asarray(history, dtype=np.int32)
    names_rows = bool(tokens.size) and int(tokens.min()) < 0
    if names_rows and int(tokens.min()) < -fed_rows:
        raise ValueError(
            f"a history names sampling row {-int(tokens.min()) - 1} of the step before, which left {fed_rows}"
        )
    return np.concatenate([params.reshape(-1), tokens]), 8 * n, any_penalty, names_rows


class Sampler:
    def __init__(self, device: torch.device | str = "cuda") -> None:
        self.device = torch.device(device)

    def _index(self, row_index: Sequence[int] | None) -> torch.Tensor | None:
        if row_index is None:
            return None
        return upload_ints(list(row_index), self.device)

    def sample(
        self,
        logits: torch.Tensor,
        rows: Sequence[RowSampling],
        want_logprobs: bool = False,
        row_index: Sequence[int] | None = None,
        out: torch.Tensor | None = None,
        fed: torch.Tensor | None = None,
    ) -> tuple[torch.Tensor, torch.Tensor | None]:
        """``logits [R, vocab]`` float32 -> chosen ids ``[n]`` int32 (on the device) and,
        if asked, the chosen tokens' log-probabilities ``[n]`` float32.  Sampling row ``b``
        reads row ``row_index[b]`` of the logits; without an index there is one sampling
        row per row of logits, in order.  ``out`` (int32, at least ``n`` long) receives the
        ids in place of a new tensor.  ``fed`` (int32) holds the choices of the step before,
        for the histories that name its rows; it is not ``out``.  Nothing here waits for the
        device."""
        n = len(rows)
        reads = len(row_index) if row_index is not None else logits.shape[0]
        if n != reads:
            raise ValueError(f"{reads} rows of logits for {n} sampling rows")
        if out is None:
            out = torch.empty(n, dtype=torch.int32, device=self.device)
        elif out.numel() < n:
            raise ValueError(f"{n} sampling rows do not fit an output of {out.numel()}")
        else:
            out = out[:n]
        if n == 0:
            return out, (torch.empty(0, dtype=torch.float32, device=self.device) if want_logprobs else None)
        index = self._index(row_index)
        plain = all(r.temperature == 0.0 and r.repetition_penalty == 1.0 for r in rows)
        if plain and not want_logprobs:
            ops.argmax(logits, out, index)
            return out, None
        packed, words, any_penalty, names_rows = _pack_rows(rows, 0 if fed is None else fed.numel())
        dev = upload(packed, self.device)
        logprob = torch.empty(n, dtype=torch.float32, device=self.device) if want_logprobs else None
        ops.sample(
            logits, dev[:words], dev[words:] if any_penalty else None, out, logprob, any_penalty, index,
            fed if names_rows else None,
        )
        return out, logprob

    def logprobs(
        self,
        logits: torch.Tensor,
        targets: torch.Tensor | Sequence[int],
        k: int,
        rows: Sequence[RowSampling] | None = None,
        row_index: Sequence[int] | None = None,
        fed: torch.Tensor | None = None,
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """Log-probability of ``targets[b]`` and the ``k`` most likely tokens, on the device:
        ``(target [n], top ids [n, k], top log-probabilities [n, k])``.

        With ``rows`` the distribution is the one those rows are sampled from, penalty and
        temperature applied, a greedy row at temperature 1 (rapid_llm/engine/sampler.py:
        698-716).  Without, the raw logits are scored, as for the tokens of a prompt
        (:425-447)."""
        if not isinstance(targets, torch.Tensor):
            targets = upload_ints(list(targets), self.device)
        elif targets.device != self.device or targets.dtype != torch.int32:
            targets = targets.to(device=self.device, dtype=torch.int32)
        n = targets.shape[0]
        if rows is not None and len(rows) != n:
            raise ValueError(f"{n} targets for {len(rows)} sampling rows")
        index = self._index(row_index)
        if rows is None:
            return ops.logprobs(logits, targets, k, row_index=index)
        packed, words, any_penalty, names_rows = _pack_rows(rows, 0 if fed is None else fed.numel())
        dev = upload(packed, self.device)
        return ops.logprobs(
            logits, targets, k, dev[:words], dev[words:] if any_penalty else None, any_penalty, index,
            fed if names_rows else None,
        )


def to_records(
    token_ids: Sequence[int],
    ks: Sequence[int | None],
    target_lp: Sequence[float],
    top_ids: Sequence[Sequence[int]],
    top_lp: Sequence[Sequence[float]],
) -> list[PositionLogprobs | None]:
    """Host lists of one batch -> one record per row, ``None`` where none was asked for
    (rapid_llm/engine/sampler.py:388-422).  Row ``b`` keeps the first ``ks[b]`` of the
    alternatives; places the kernel marked empty (id -1) are dropped."""
    records: list[PositionLogprobs | None] = []
    for b, k in enumerate(ks):
        if k is None:
            records.append(None)
            continue
        ids = [i for i in top_ids[b][:k] if i >= 0] if k else []
        records.append(
            PositionLogprobs(
                token_id=int(token_ids[b]),
                logprob=float(target_lp[b]),
                top_token_ids=tuple(int(i) for i in ids),
                top_logprobs=tuple(float(v) for v in top_lp[b][: len(ids)]),
            )
        )
    return records
