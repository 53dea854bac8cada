"""Decoding parameters of one request.

Names, meanings and validation are the reference's (rapid_llm/engine/sampler.py:44-97).
Two departures: ``seed`` is new (the reference draws from the process-wide generator,
:218,:243, so a request's tokens depend on what else was sampled before it; here every
request has its own counter-based stream), and the defaults of ``repetition_penalty`` and
``stop_on_repeat`` are the neutral ones, so that a default request is reproducible from
its logits alone.
"""

from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 0.6  # 0 means greedy (arg-max)
    top_p: float = 0.9  # nucleus threshold in (0, 1]
    max_gen_len: int | None = None  # None: fill the remaining context window
    repetition_penalty: float = 1.0  # over generated tokens; 1.0 disables it
    stop_on_repeat: bool = False  # engine-side breaker of repeating output
    logprobs: int | None = None  # per generated token: its log-probability and the k most likely
    prompt_logprobs: int | None = None  # the same for the prompt's own tokens (position 0 has none)
    seed: int | None = None  # None: derived from the engine's seed and the request's number
    ignore_eos: bool = False  # keep generating through stop tokens (benchmarks)

    def __post_init__(self) -> None:
        if self.temperature < 0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")
        if self.max_gen_len is not None and self.max_gen_len < 1:
            raise ValueError(f"max_gen_len must be >= 1 or None, got {self.max_gen_len}")
        if self.repetition_penalty <= 0:
            raise ValueError(f"repetition_penalty must be > 0, got {self.repetition_penalty}")
        for name in ("logprobs", "prompt_logprobs"):
            value = getattr(self, name)
            if value is not None and value < 0:
                raise ValueError(f"{name} must be >= 0, got {value}")
        if self.seed is not None and not 0 <= self.seed < 1 << 64:
            raise ValueError(f"seed must fit 64 unsigned bits, got {self.seed}")

    @property
    def is_greedy(self) -> bool:
        return self.temperature == 0.0
