"""Log-probability records of a position (rapid_llm/engine/sampler.py:112-131)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class PositionLogprobs:
    """The token at one position and the best alternatives there.

    ``logprob`` is the token's log-probability under the distribution the position
    produced; the token need not be among the ``k`` most likely ones listed beside it
    (descending, equal values by ascending id)."""

    token_id: int
    logprob: float
    top_token_ids: tuple[int, ...] = ()
    top_logprobs: tuple[float, ...] = ()
