"""Continuous batching above the step function: admit, cut prompts into portions under a
token budget, decode, finish and free.

Every call of :meth:`Scheduler.step` plans one batch and runs it as ONE forward pass:
single decoded tokens of some requests beside prompt portions of others.  The reference
plans the same sets but runs them as up to three passes (rapid_llm/engine/scheduler.py:
964-988); its planning rules are kept (rapid_llm/engine/batch_planner.py):

* requests are admitted first come, first served, while a slot, the pages of the first
  portion and token budget are there (:579-666); a request that does not fit waits, and
  nobody overtakes it;
* a portion is ``min(remaining, max_chunk_size, budget)`` tokens (:683-698); running
  requests' portions are served before new admissions (:485-504); a portion that cannot get
  pages keeps its slot and progress and tries again next step (:496-499);
* the budget counts the true tokens of the step, decoded tokens included (the reference
  prices a padded grid, :600-610; nothing is padded here);
* the request whose last uncomputed token runs in a step is sampled in that step and
  decodes from the next one (:509-518).

**When pages run out** (:536-552,:972-1023).  A decoding request that cannot get the page
for its next token evicts the youngest running request that has no work in this step yet;
if there is none, it is evicted itself, unless it is the only request left, in which case
the pool is simply too small for it and it finishes with reason ``"length"``.  If all
running requests are stuck in their prompts, the youngest is evicted so that the others can
go on.  Eviction is recomputation: slot and pages are given back, progress is reset to
zero, and the request returns to the *front* of the queue; its generated tokens are kept
and run again as if they were prompt, and because the i-th draw of a request depends only
on its seed and i, it continues with exactly the tokens it would have produced.

**The launch/harvest pipeline** (:818-933; on unless ``EngineConfig.pipeline`` or the
environment variable ``RAPID_LLM_PIPELINE`` says otherwise).  ``step`` queues step N + 1 on
the device before it reads what step N chose, so planning, packing and the harvest itself
run while the device computes.  A request sampled in step N owns a *pending* token until the
harvest: it counts in the request's length, and step N + 1 feeds it from the device
(:func:`~rapid_llm_amd.engine.feed.fed_token`).  Ends that depend on counts (``max_gen_len``,
``max_seq_len``) are known when planning and cost nothing.  Ends that depend on the token
(a stop token, the repetition breaker) are seen one step late: the request has then ridden
one more step, whose token is discarded, and its slot and pages are given back after that
step.  Nobody is evicted or ended for want of pages on a guess: when pages are short, the
step in flight is read first and the decision made on what is then known.  The tokens are
those of the synchronous loop, with a repetition penalty too: the history of a request whose
newest token is pending names that token by its sampling row, and the sampling kernels read
it on the device.
"""

from __future__ import annotations

import itertools
import os
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Any, Iterable, Sequence

from ..config.engine_config import EngineConfig
from ..sampling.logprobs import PositionLogprobs
from ..sampling.params import SamplingParams
from ..sampling.rng import derive_seed
from .feed import fed_token
from .request import Request, RequestStatus

# Output tokens of a request between checks of the repetition breaker.  The reference polls
# every 8th step of the engine (scheduler.py:1414); counting the request's own tokens makes
# the end of a request independent of what else runs and of the pipeline.
REPEAT_POLL_INTERVAL = 8


@dataclass
class Work:
    """One request's share of a step: tokens ``[start, start + count)`` of its sequence."""

    request: Request
    start: int
    count: int
    samples: bool  # the portion ends the sequence so far: its last logits choose a token


@dataclass
class StepPlan:
    work: list[Work] = field(default_factory=list)
    preempted: list[Request] = field(default_factory=list)
    finished: list[Request] = field(default_factory=list)  # ended by the planner (pool too small)

    @property
    def num_tokens(self) -> int:
        return sum(w.count for w in self.work)


@dataclass
class SamplingPlan:
    """What is to be read off the logits of one step.  The step returns one row of logits
    per wanted place, in the order of the entries and of their ``want``."""

    rows: list = field(default_factory=list)  # RowSampling, one per token to choose
    logits_rows: list[int] = field(default_factory=list)  # the row of logits each reads
    logprob_ks: list[int | None] = field(default_factory=list)  # per chosen token: alternatives to report
    # prompt positions to score: row of logits, the token that follows there, alternatives
    prompt_rows: list[int] = field(default_factory=list)
    prompt_targets: list[int] = field(default_factory=list)
    prompt_ks: list[int] = field(default_factory=list)


@dataclass
class StepOutput:
    token_ids: list[int]  # parallel to SamplingPlan.rows
    logprobs: list[PositionLogprobs | None] | None = None  # parallel to rows, if any asked
    prompt_logprobs: list[PositionLogprobs] | None = None  # parallel to prompt_rows


class _ReadFirst(Exception):
    """Planning met a shortage of pages while a step is in flight."""


class _Done:
    """The handle of a step that an executor without ``launch`` has already run."""

    def __init__(self, output: StepOutput) -> None:
        self._output = output

    def result(self) -> StepOutput:
        return self._output


@dataclass
class _Inflight:
    handle: Any  # .result() -> StepOutput
    sampled: list[Request]  # parallel to the sampling rows of the step
    scored: list[tuple[Request, int]]  # (request, prompt position) parallel to its prompt rows


def detect_repetition(token_ids: Sequence[int], window: int = 32, min_reps: int = 3) -> bool:
    """Whether the output ends in a block of ``window`` tokens that occurred at least
    ``min_reps`` times before.  The reference applies the same test to the last 128
    characters of the text (rapid_llm/engine/stop_criteria.py:63-77); token ids are used
    here so that it works without a tokenizer."""
    n = len(token_ids)
    if n < window * (min_reps + 1):
        return False
    recent = list(token_ids[-window:])
    seen = 0
    for start in range(0, n - 2 * window + 1):
        if token_ids[start] == recent[0] and list(token_ids[start : start + window]) == recent:
            seen += 1
            if seen >= min_reps:
                return True
    return False


class Scheduler:
    """``executor`` owns the model side.  It has ``cache`` (the
    :class:`~rapid_llm_amd.cache.manager.CacheManager` whose slots and pages the plan takes),
    ``execute(entries, sampling: SamplingPlan) -> StepOutput`` running one step, choosing
    a token for every row of the plan and scoring what it asks to be scored, and
    ``finish(request_id)`` giving back what a request holds."""

    def __init__(
        self,
        executor: Any,
        config: EngineConfig,
        stop_token_ids: Iterable[int] = (),
        tokenizer: Any = None,
    ) -> None:
        self.executor = executor
        self.cache = executor.cache
        self.config = config
        self.stop_token_ids = frozenset(int(t) for t in stop_token_ids)
        self.tokenizer = tokenizer
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self._ids = itertools.count()
        self._admissions = itertools.count()
        self._requests: dict[str, Request] = {}
        self._detok: dict[str, Any] = {}
        self._step_count = 0
        self.num_preemptions = 0
        self.last_plan: StepPlan | None = None
        pipeline = getattr(config, "pipeline", None)
        if pipeline is None:  # the reference's switch (rapid_llm/executor/worker.py:50-53), on by default here
            pipeline = os.environ.get("RAPID_LLM_PIPELINE", "1").strip().lower() in ("1", "true", "on")
        self.pipeline = bool(pipeline) and hasattr(executor, "launch")
        self._inflight: _Inflight | None = None
        self._held: list[Request] = []  # finished, but a step in flight still uses their slot and pages

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_pretrained(
        cls,
        model,
        *,
        tokenizer=None,
        max_seq_len: int = 2048,
        max_num_seqs: int = 32,
        max_num_batched_tokens: int = 8192,
        enable_chunked_prefill: bool = True,
        max_chunk_size: int = 512,
        max_gpu_num_blocks: int | None = None,
        device: str = "cuda",
        use_cuda_graph: bool = True,
        dtype: str = "bfloat16",
        page_size: int = 16,
        num_pages: int | None = None,
        load_format: str = "auto",
        seed: int = 0,
        hf_overrides=None,
        pipeline: bool | None = None,
    ) -> "Scheduler":
        """Names and defaults of rapid_llm/engine/scheduler.py:409-440 where it has them."""
        from .llm import build_engine

        return build_engine(
            model, tokenizer=tokenizer, max_seq_len=max_seq_len, max_num_seqs=max_num_seqs,
            max_num_batched_tokens=max(max_num_batched_tokens, 0 if enable_chunked_prefill else max_seq_len),
            max_chunk_size=max_chunk_size if enable_chunked_prefill else 0,
            max_gpu_num_blocks=max_gpu_num_blocks, device=device, use_cuda_graph=use_cuda_graph,
            dtype=dtype, page_size=page_size, num_pages=num_pages, load_format=load_format,
            seed=seed, hf_overrides=hf_overrides, pipeline=pipeline,
        )

    # ------------------------------------------------------------------ submission
    def add_request(
        self,
        prompt: str | Sequence[int],
        params: SamplingParams | None = None,
        request_id: str | None = None,
    ) -> Request:
        """rapid_llm/engine/batch_planner.py:403-427: unique id, no empty prompt, the prompt
        must leave room for one token, ``max_new_tokens`` is capped by the context."""
        params = params or SamplingParams()
        number = next(self._ids)
        if request_id is None:
            request_id = f"req-{number}"
        if request_id in self._requests:  # finished requests are not kept: the id is free again
            raise ValueError(f"request id {request_id!r} is already in use")
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer; pass token ids instead")
            text, ids = prompt, list(self.tokenizer.encode(prompt))
        else:
            text, ids = None, [int(t) for t in prompt]
        if not ids:
            raise ValueError("empty prompt")
        limit = self.config.max_seq_len
        if len(ids) >= limit:
            raise ValueError(f"prompt of {len(ids)} tokens leaves no room under max_seq_len {limit}")
        capacity = self.cache.capacity_tokens()
        if len(ids) + 1 > capacity:
            raise ValueError(
                f"prompt of {len(ids)} tokens does not fit the cache pool of {capacity} tokens"
            )
        room = limit - len(ids)
        max_new = room if params.max_gen_len is None else min(params.max_gen_len, room)
        request = Request(
            request_id=request_id,
            prompt=text,
            prompt_token_ids=ids,
            params=params,
            max_new_tokens=max_new,
            seed=params.seed if params.seed is not None else derive_seed(self.config.seed, number),
        )
        if params.logprobs is not None:
            request.output_logprobs = []
        self._requests[request_id] = request
        self.waiting.append(request)
        if self.tokenizer is not None:
            from .tokenizer import Detokenizer

            self._detok[request_id] = Detokenizer(self.tokenizer)
        return request

    def abort(self, request_id: str) -> None:
        request = self._requests.get(request_id)
        if request is None or request.is_finished:
            return
        self._finish(request, "abort")

    def has_unfinished_requests(self) -> bool:
        return bool(self.waiting or self.running or self._inflight is not None)

    # ------------------------------------------------------------------ bookkeeping
    def _finish(self, request: Request, reason: str) -> None:
        """A token of the request that is still in flight belongs to nobody: the request
        stopped before it.  Slot and pages are given back when that step has been read."""
        if request.status is RequestStatus.RUNNING:
            self.running.remove(request)
            if request.pending:
                self._held.append(request)  # given back when the step in flight has been read
            else:
                self.executor.finish(request.request_id)
        elif request.status is RequestStatus.WAITING:
            self.waiting.remove(request)
        request.discard = request.pending
        request.status = RequestStatus.FINISHED
        request.finish_reason = reason
        request.finish_time = time.monotonic()
        self._detok.pop(request.request_id, None)
        # the caller holds the request object; the engine keeps nothing of a finished request
        self._requests.pop(request.request_id, None)

    def _preempt(self, request: Request, plan: StepPlan) -> None:
        """Eviction by recomputation (rapid_llm/engine/batch_planner.py:987-1023)."""
        self.running.remove(request)
        self.executor.finish(request.request_id)
        request.status = RequestStatus.WAITING
        request.num_computed_tokens = 0
        request.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(request)
        plan.preempted.append(request)

    def _ends_at_harvest(self, request: Request) -> bool:
        """The token in flight is the request's last, by count: it is not planned further."""
        return request.pending > 0 and (
            not request.has_room or request.seq_len >= self.config.max_seq_len
        )

    def _portion(self, request: Request, budget: int) -> int:
        """Tokens of the request's next portion under what is left of the budget
        (rapid_llm/engine/batch_planner.py:683-698); 0 when it has to wait."""
        remaining = request.num_uncomputed
        if self.config.max_chunk_size == 0:  # chunking off: whole or not at all
            return remaining if remaining <= budget else 0
        return min(remaining, self.config.max_chunk_size, budget)

    # ------------------------------------------------------------------ planning
    def plan(self) -> StepPlan:
        plan = StepPlan()
        cache = self.cache
        budget = self.config.max_num_batched_tokens
        granted: set[str] = set()

        # 1. decoding requests, oldest first; each needs room for one more position
        for request in sorted(self.running, key=lambda r: r.admission_number):
            if request.status is not RequestStatus.RUNNING or request.num_uncomputed != 1:
                continue
            if self._ends_at_harvest(request):
                continue
            if budget < 1:
                break
            rid = request.request_id
            while not cache.reserve(rid, request.seq_len, request.num_computed_tokens):
                if self._inflight is not None:
                    raise _ReadFirst  # the step in flight may end requests and free their pages
                victims = [
                    r for r in self.running if r is not request and r.request_id not in granted
                ]
                if victims:
                    self._preempt(max(victims, key=lambda r: r.admission_number), plan)
                    continue
                if len(self.running) > 1:
                    self._preempt(request, plan)  # the others will leave pages behind
                else:
                    self._finish(request, "length")  # alone, and the pool is exhausted
                    plan.finished.append(request)
                break
            else:
                plan.work.append(Work(request, request.num_computed_tokens, 1, True))
                granted.add(rid)
                budget -= 1

        # 2. running requests still in their prompt (or recomputing after an eviction)
        for request in sorted(self.running, key=lambda r: r.admission_number):
            if request.request_id in granted or request.num_uncomputed <= 1:
                continue
            count = self._portion(request, budget)
            if count < 1:
                continue
            start = request.num_computed_tokens
            if not cache.reserve(request.request_id, start + count, start):
                continue  # keeps slot and progress, tries again next step
            plan.work.append(Work(request, start, count, count == request.num_uncomputed))
            granted.add(request.request_id)
            budget -= count

        # 3. admissions, first come first served
        while self.waiting and len(self.running) < self.config.max_num_seqs and not plan.preempted:
            request = self.waiting[0]
            count = self._portion(request, budget)
            if count < 1:
                break
            if cache.has(request.request_id):
                # the id's previous request has ended, but a step in flight still rides on its
                # slot and pages: the new one waits the one step until they are given back
                break
            if cache.admit(request.request_id) is None:
                break
            if not cache.reserve(request.request_id, count, 0):
                cache.release(request.request_id)  # nothing was taken but the slot
                break
            self.waiting.popleft()
            request.status = RequestStatus.RUNNING
            request.admission_number = next(self._admissions)
            request.scheduled_time = time.monotonic()
            self.running.append(request)
            plan.work.append(Work(request, 0, count, count == request.num_uncomputed))
            granted.add(request.request_id)
            budget -= count
        return plan

    def _plan_with_progress(self) -> StepPlan:
        """A plan that runs something whenever anything can run."""
        plan = self.plan()

        def stuck() -> list[Request]:
            # running requests that have work and got none: they wait for pages
            return [r for r in self.running if not self._ends_at_harvest(r)]

        while not plan.work and stuck():
            if self._inflight is not None:
                raise _ReadFirst
            youngest = max(stuck(), key=lambda r: r.admission_number)
            if len(self.running) == 1:
                self._finish(youngest, "length")
                plan.finished.append(youngest)
            else:
                self._preempt(youngest, plan)
            more = self.plan()
            more.preempted = plan.preempted + more.preempted
            more.finished = plan.finished + more.finished
            plan = more
        if (
            not plan.work and not plan.finished and self.waiting and not self.running
            and self._inflight is None and not self._held
        ):
            raise RuntimeError(
                f"request {self.waiting[0].request_id!r} cannot be admitted into an empty engine"
            )
        return plan

    # ------------------------------------------------------------------ the loop
    def step(self) -> list[Request]:
        """Plan one batch, run it, harvest chosen tokens.  Returns the requests that advanced
        or finished (rapid_llm/engine/scheduler.py:1405-1460).  Pipelined, the tokens harvested
        are those of the step queued by the previous call (:818-933)."""
        if self.pipeline:
            try:
                launched, advanced = self._launch()
            except _ReadFirst:
                # pages are short: who is evicted or ended is decided on what is known, after
                # the step in flight has been read (nothing was decided or queued so far)
                advanced = self._harvest(self._inflight)
                self._inflight = None
                launched, ended = self._launch()
                advanced += ended
            else:
                if self._inflight is not None:
                    advanced += self._harvest(self._inflight)
            self._inflight = launched
            return advanced
        advanced = []
        if self._inflight is not None:  # leaving the pipeline: read what is in flight first
            advanced += self._harvest(self._inflight)
            self._inflight = None
        launched, ended = self._launch()
        advanced += ended
        if launched is not None:
            advanced += self._harvest(launched)
        return advanced

    @staticmethod
    def _penalised_tokens(request: Request) -> Sequence[int]:
        """The generated tokens a repetition penalty applies to; the one still on the device is
        named by the sampling row that chose it."""
        if request.params.repetition_penalty == 1.0:
            return ()
        if request.pending:
            return [*request.output_token_ids, fed_token(request.pending_row)]
        return request.output_token_ids

    def _launch(self) -> tuple["_Inflight | None", list[Request]]:
        """Plan a step and queue it; returns what is in flight and the requests the planner
        ended."""
        from ..sampling.sampler import RowSampling
        from .step import StepEntry

        plan = self._plan_with_progress()
        self.last_plan = plan
        self._step_count += 1
        if not plan.work:
            return None, list(plan.finished)
        entries, sampled = [], []
        sampling = SamplingPlan()
        scored: list[tuple[Request, int]] = []  # (request, prompt position the record is for)
        num_rows = 0
        for w in plan.work:
            r = w.request
            p = r.params
            want: list[int] = []
            if p.prompt_logprobs is not None:
                # the logits at position q score the prompt's token q + 1
                # (rapid_llm/engine/scheduler.py:143-148); what an earlier run of these
                # positions has scored (before an eviction) is not scored again
                if r.prompt_logprobs is None:
                    r.prompt_logprobs = [None] * r.prompt_len
                for j in range(w.count):
                    q = w.start + j + 1
                    if q < r.prompt_len and r.prompt_logprobs[q] is None:
                        sampling.prompt_rows.append(num_rows + len(want))
                        sampling.prompt_targets.append(r.prompt_token_ids[q])
                        sampling.prompt_ks.append(p.prompt_logprobs)
                        scored.append((r, q))
                        want.append(j)
            if w.samples:
                sampling.rows.append(
                    RowSampling(
                        temperature=p.temperature,
                        top_p=p.top_p,
                        repetition_penalty=p.repetition_penalty,
                        seed=r.seed,
                        counter=len(r.output_token_ids) + r.pending,
                        generated=self._penalised_tokens(r),
                    )
                )
                sampling.logits_rows.append(num_rows + len(want))
                sampling.logprob_ks.append(p.logprobs)
                sampled.append(r)
                want.append(w.count - 1)
            entries.append(StepEntry(r.request_id, r.tokens(w.start, w.start + w.count), want))
            num_rows += len(want)
        if hasattr(self.executor, "launch"):
            handle = self.executor.launch(entries, sampling)
        else:
            handle = _Done(self.executor.execute(entries, sampling))
        # the plan is committed (rapid_llm/engine/batch_planner.py:462-470)
        for w in plan.work:
            w.request.num_computed_tokens = w.start + w.count
            self.cache.trim(w.request.request_id, w.request.num_computed_tokens)
        for row, request in enumerate(sampled):
            request.pending += 1
            request.pending_row = row
        return _Inflight(handle, sampled, scored), list(plan.finished)

    def _harvest(self, inflight: "_Inflight") -> list[Request]:
        """Read a step's tokens back and retire whoever stopped
        (rapid_llm/engine/scheduler.py:1405-1460)."""
        result = inflight.handle.result()
        tokens, logprobs = result.token_ids, result.logprobs
        for (request, q), record in zip(inflight.scored, result.prompt_logprobs or ()):
            request.prompt_logprobs[q] = record
        now = time.monotonic()
        advanced: list[Request] = []
        for i, request in enumerate(inflight.sampled):
            token = int(tokens[i])
            request.pending -= 1
            if request.discard:
                # the request stopped at an earlier harvest: this token belongs to nobody
                request.discard -= 1
                continue
            request.delta = ""
            if request.first_token_time is None:
                request.first_token_time = now
            advanced.append(request)
            if token in self.stop_token_ids and not request.params.ignore_eos:
                # the stop token is punctuation, not output (scheduler.py:1430-1436)
                self._finish(request, "eos")
                continue
            request.output_token_ids.append(token)
            if request.output_logprobs is not None and logprobs is not None:
                request.output_logprobs.append(logprobs[i])
            detok = self._detok.get(request.request_id)
            if detok is not None:
                piece = detok.append(token)
                request.delta = piece
                request.text += piece
            outputs = len(request.output_token_ids)
            if outputs >= request.max_new_tokens or request.prompt_len + outputs >= self.config.max_seq_len:
                self._finish(request, "length")
            elif (
                request.params.stop_on_repeat
                and outputs % REPEAT_POLL_INTERVAL == 0
                and detect_repetition(request.output_token_ids)
            ):
                self._finish(request, "repeat")
        held = []
        for request in self._held:
            if request.pending:
                held.append(request)
            else:
                self.executor.finish(request.request_id)
        self._held = held
        return advanced

    def run_to_completion(self) -> None:
        while self.has_unfinished_requests():  # rapid_llm/engine/scheduler.py:1322-1323
            self.step()
