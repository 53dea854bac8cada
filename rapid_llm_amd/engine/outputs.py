"""What ``LLM.generate`` returns (rapid_llm/engine/outputs.py:21-59), plus the token ids,
which are all a model with random weights and no tokenizer can give."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..sampling.logprobs import PositionLogprobs


@dataclass
class CompletionOutput:
    index: int
    text: str
    finish_reason: str | None
    token_ids: list[int] = field(default_factory=list)
    logprobs: list[PositionLogprobs] | None = None  # parallel to token_ids, if asked


@dataclass
class RequestOutput:
    prompt: str | None
    outputs: list[CompletionOutput]
    prompt_token_ids: list[int] = field(default_factory=list)
    request_id: str = ""
    # per prompt position, if asked; position 0 has no predictor and is None
    prompt_logprobs: list[PositionLogprobs | None] | None = None

    @property
    def text(self) -> str:
        return self.outputs[0].text

    @property
    def token_ids(self) -> list[int]:
        return self.outputs[0].token_ids
