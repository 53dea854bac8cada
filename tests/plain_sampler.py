"""Plain token selection, the oracle of the sampling kernel.  Shares no code with the engine.

The order of operations is the reference's ``Sampler._draw`` (rapid_llm/engine/sampler.py:
641-718): repetition penalty, then greedy rows take the arg-max, other rows the softmax of
``logits / temperature`` and a nucleus draw.  The reference draws with ``torch.multinomial``
from the process-wide generator; here the draw is the inverse of the cumulative distribution
at a given ``u`` in [0, 1), which is what a seeded engine can be compared with.
"""

from __future__ import annotations

import torch

POOL = 1024  # rapid_llm/engine/sampler.py:186 (_TOP_P_CANDIDATES)


def plain_repetition_penalty(logits: torch.Tensor, generated: list[int], penalty: float) -> torch.Tensor:
    """Every token that was generated, once: a negative logit is multiplied by the penalty,
    any other divided (rapid_llm/engine/sampler.py:134-179)."""
    out = logits.clone()
    for tok in set(generated):
        out[tok] = out[tok] * penalty if out[tok] < 0 else out[tok] / penalty
    return out


def plain_nucleus(probs: torch.Tensor, top_p: float, pool: int = POOL) -> tuple[torch.Tensor, torch.Tensor]:
    """The candidates in descending order and their kept probabilities (not renormalised).

    ``topk`` over a pool of ``pool`` (rapid_llm/engine/sampler.py:209-221); a candidate is
    dropped when the mass *before* it exceeds ``top_p``, but only if the pool reaches
    ``top_p`` at all (:234-244)."""
    k = min(pool, probs.numel())
    # descending by probability, ties by lower index (a stable sort fixes what topk leaves open)
    order = torch.sort(probs, descending=True, stable=True).indices[:k]
    top = probs[order].clone()
    cum = torch.cumsum(top, dim=0)
    drop = (cum - top) > top_p
    if not bool(cum[-1] > top_p):
        drop[:] = False
    top[drop] = 0.0
    return order, top


def plain_sample(
    logits: torch.Tensor,
    temperature: float,
    top_p: float,
    u: float,
    penalty: float = 1.0,
    generated: list[int] = (),
) -> int:
    logits = logits.to(torch.float32)
    if penalty != 1.0 and len(generated):
        logits = plain_repetition_penalty(logits, list(generated), penalty)
    if temperature == 0.0:
        return int(torch.argmax(logits))  # rapid_llm/engine/sampler.py:95-97
    probs = torch.softmax(logits / temperature, dim=-1)
    if top_p == 1.0:
        ids, kept = torch.arange(probs.numel()), probs  # :218: the whole distribution
    else:
        ids, kept = plain_nucleus(probs, top_p)
    cum = torch.cumsum(kept.double(), dim=0)
    target = u * float(cum[-1])
    below = int((cum < target).sum())
    # the first token whose cumulative mass reaches the target; never one with zero mass
    nz = torch.nonzero(kept > 0).flatten()
    j = min(below, int(nz[-1]))
    return int(ids[j])


def plain_logprob(logits: torch.Tensor, token: int, temperature: float, penalty: float = 1.0,
                  generated: list[int] = ()) -> float:
    logits = logits.to(torch.float32)
    if penalty != 1.0 and len(generated):
        logits = plain_repetition_penalty(logits, list(generated), penalty)
    t = temperature if temperature > 0 else 1.0  # rapid_llm/engine/sampler.py:508
    return float(torch.log_softmax(logits.double() / t, dim=-1)[token])


def plain_top_logprobs(logits: torch.Tensor, k: int, temperature: float = 1.0, penalty: float = 1.0,
                       generated: list[int] = ()) -> tuple[list[int], list[float]]:
    """The ``k`` most likely tokens and their log-probabilities, descending, equal values by
    ascending id: ``log_softmax`` of the final logits, then ``topk``
    (rapid_llm/engine/sampler.py:362-369).  The raw logits with the defaults, as a prompt is
    scored (:425-447)."""
    logits = logits.to(torch.float32)
    if penalty != 1.0 and len(generated):
        logits = plain_repetition_penalty(logits, list(generated), penalty)
    t = temperature if temperature > 0 else 1.0
    z = logits / t
    lp = torch.log_softmax(z.double(), dim=-1)
    order = torch.sort(z, descending=True, stable=True).indices[:k]
    return order.tolist(), lp[order].tolist()
