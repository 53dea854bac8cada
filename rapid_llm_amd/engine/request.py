"""One generation request, from arrival to completion.

Field names follow the reference's ``Request`` (rapid_llm/engine/batch_planner.py:25-150).
The tokens a request has to run are ``prompt_token_ids + output_token_ids``;
``num_computed_tokens`` of them are in the cache.  Whenever a step brings the last of
them, the logits at that place choose the next token.  A prompt portion, a decoded token
and the recomputation after an eviction are therefore the same thing: the next
``n`` uncomputed tokens.

Under the launch/harvest pipeline a request may own one token that the device has chosen
and the host has not read yet (``pending``, rapid_llm/engine/scheduler.py:214-262): it
counts as part of the sequence, and where its id is needed the placeholder of the sampling
row that chose it stands (``pending_row``).
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from enum import Enum

from ..sampling.logprobs import PositionLogprobs
from ..sampling.params import SamplingParams
from .feed import fed_token


class RequestStatus(str, Enum):
    WAITING = "waiting"  # holds no slot and no pages
    RUNNING = "running"  # holds one slot
    FINISHED = "finished"


@dataclass
class Request:
    request_id: str
    prompt: str | None
    prompt_token_ids: list[int]
    params: SamplingParams
    max_new_tokens: int = 0
    seed: int = 0
    num_computed_tokens: int = 0
    arrival_time: float = field(default_factory=time.monotonic)
    scheduled_time: float | None = None
    admission_number: int = -1  # order of the latest admission: larger is younger
    status: RequestStatus = RequestStatus.WAITING
    output_token_ids: list[int] = field(default_factory=list)
    output_logprobs: list[PositionLogprobs] | None = None  # parallel to output_token_ids, if asked
    prompt_logprobs: list[PositionLogprobs | None] | None = None  # per prompt position; [0] is None
    text: str = ""
    delta: str = ""
    finish_reason: str | None = None  # "eos" | "length" | "repeat" | "abort"
    first_token_time: float | None = None
    finish_time: float | None = None
    num_preemptions: int = 0
    pending: int = 0  # tokens chosen on the device that the host has not read yet (0 or 1)
    pending_row: int = -1  # the sampling row of the step in flight that chooses the pending token
    discard: int = 0  # pending tokens that belong to nobody: the request stopped before them

    @property
    def prompt_len(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def seq_len(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids) + self.pending

    @property
    def num_uncomputed(self) -> int:
        return self.seq_len - self.num_computed_tokens

    @property
    def is_finished(self) -> bool:
        return self.status is RequestStatus.FINISHED

    @property
    def has_room(self) -> bool:
        return len(self.output_token_ids) + self.pending < self.max_new_tokens

    @property
    def prefill_done(self) -> bool:
        """Everything but the newest token is in the cache: the next step is a decode."""
        return self.num_uncomputed <= 1 and bool(self.output_token_ids or self.pending)

    def tokens(self, start: int, stop: int) -> list[int]:
        """Tokens ``[start, stop)`` of the sequence; a pending token is named by the
        placeholder of the sampling row that chooses it."""
        n = len(self.prompt_token_ids)
        m = n + len(self.output_token_ids)
        out: list[int] = []
        if start < n:
            out += self.prompt_token_ids[start : min(stop, n)]
        if stop > n and start < m:
            out += self.output_token_ids[max(start, n) - n : min(stop, m) - n]
        if stop > m:
            out += [fed_token(self.pending_row)] * (stop - max(start, m))
        return out
