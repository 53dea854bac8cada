"""The Python entry point: ``LLM(model).generate(prompts, SamplingParams(...))``.

Constructor names follow the reference's ``LLM`` (rapid_llm/engine/llm.py:78-97) where it
has them; what it offers beyond one GPU and one architecture (quantisation, parallel sizes,
images) has no counterpart here and is refused by name rather than ignored.  ``generate``
drives the continuous-batching :class:`~rapid_llm_amd.engine.scheduler.Scheduler`; the
reference's ``LLM`` drives a static batch (rapid_llm/engine/llm_engine.py:70-269) and keeps
the scheduler for its server.  Prompts may be strings (the model folder then needs a
``tokenizer.json``) or lists of token ids.
"""

from __future__ import annotations

from pathlib import Path
from typing import Any, Iterator, Mapping, Sequence

import numpy as np
import torch

from ..config.engine_config import EngineConfig
from ..sampling.params import SamplingParams
from ..kernels.upload import upload_ints
from ..sampling.sampler import Sampler, to_records
from .outputs import CompletionOutput, RequestOutput
from .request import Request
from .scheduler import SamplingPlan, Scheduler, StepOutput


class PendingStep:
    """A step that has been queued on the device.  ``result()`` waits for it and returns its
    :class:`StepOutput`; until then the host is free to plan and queue the next step."""

    def __init__(self, sampling: SamplingPlan, host: dict[str, torch.Tensor], asked: list[int]) -> None:
        self._sampling = sampling
        self._host = host  # pinned copies of what the step chose and scored
        self._asked = asked
        self._event = torch.cuda.Event()
        self._event.record()
        self._output: StepOutput | None = None

    def result(self) -> StepOutput:
        if self._output is not None:
            return self._output
        # the step's one host synchronisation (rapid_llm/engine/scheduler.py:1000-1005)
        self._event.synchronize()
        sampling, host = self._sampling, self._host
        out = StepOutput(host["ids"].tolist())
        if self._asked:
            records = to_records(
                [out.token_ids[b] for b in self._asked],
                [sampling.logprob_ks[b] for b in self._asked],
                host["lp"].tolist(), host["top_ids"].tolist(), host["top_lp"].tolist(),
            )
            out.logprobs = [None] * len(out.token_ids)
            for b, record in zip(self._asked, records):
                out.logprobs[b] = record
        if sampling.prompt_rows:
            out.prompt_logprobs = to_records(
                sampling.prompt_targets, sampling.prompt_ks,
                host["p_lp"].tolist(), host["p_top_ids"].tolist(), host["p_top_lp"].tolist(),
            )
        self._output = out
        return out


class GpuExecutor:
    """The model side of the scheduler: the step function and the sampling kernels."""

    def __init__(self, runner, sampler) -> None:
        self.runner = runner
        self.sampler = sampler
        self.cache = runner.cache

    @staticmethod
    def _to_host(t: torch.Tensor) -> torch.Tensor:
        host = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
        host.copy_(t, non_blocking=True)
        return host

    def launch(self, entries, sampling: SamplingPlan) -> PendingStep:
        """Queue the step, the choice of its tokens (left in ``runner.sampled``, where the next
        step's fed tokens are read) and the copies back to the host; does not wait."""
        runner = self.runner
        logits = runner.step(entries)
        in_order = sampling.logits_rows == list(range(logits.shape[0]))
        fed = None
        if any(r.repetition_penalty != 1.0 and any(t < 0 for t in r.generated[-1:]) for r in sampling.rows):
            # a penalised row's newest token is still on the device, among the choices that
            # this step's sampling is about to overwrite
            fed = runner.sampled_before
            fed.copy_(runner.sampled)
        ids, _ = self.sampler.sample(
            logits, sampling.rows, row_index=None if in_order else sampling.logits_rows, out=runner.sampled,
            fed=fed,
        )
        host = {"ids": self._to_host(ids)}
        asked = [b for b, k in enumerate(sampling.logprob_ks) if k is not None]
        if asked:
            chosen = ids if len(asked) == len(sampling.rows) else ids[upload_ints(asked, ids.device, np.int64)]
            lp, top_ids, top_lp = self.sampler.logprobs(
                logits,
                chosen,
                max(sampling.logprob_ks[b] for b in asked),
                rows=[sampling.rows[b] for b in asked],
                row_index=[sampling.logits_rows[b] for b in asked],
                fed=fed,
            )
            host.update(lp=self._to_host(lp), top_ids=self._to_host(top_ids), top_lp=self._to_host(top_lp))
        if sampling.prompt_rows:
            lp, top_ids, top_lp = self.sampler.logprobs(
                logits, sampling.prompt_targets, max(sampling.prompt_ks), row_index=sampling.prompt_rows
            )
            host.update(p_lp=self._to_host(lp), p_top_ids=self._to_host(top_ids), p_top_lp=self._to_host(top_lp))
        return PendingStep(sampling, host, asked)

    def execute(self, entries, sampling: SamplingPlan) -> StepOutput:
        return self.launch(entries, sampling).result()

    def finish(self, request_id: str) -> None:
        self.runner.finish(request_id)


def build_engine(
    model,
    *,
    tokenizer=None,
    max_seq_len: int = 2048,
    max_num_seqs: int = 32,
    max_num_batched_tokens: int = 8192,
    max_chunk_size: int = 512,
    max_gpu_num_blocks: int | None = None,
    device: str = "cuda",
    use_cuda_graph: bool = True,
    dtype: str = "bfloat16",
    page_size: int = 16,
    num_pages: int | None = None,
    load_format: str = "auto",
    seed: int = 0,
    hf_overrides: Mapping[str, Any] | None = None,
    gpu_memory_utilization: float = 0.9,
    pipeline: bool | None = None,
) -> Scheduler:
    from .step import ModelRunner
    from .tokenizer import load_stop_token_ids, load_tokenizer

    config = EngineConfig(
        dtype=dtype,
        max_seq_len=max_seq_len,
        page_size=page_size,
        num_pages=num_pages,
        max_gpu_num_blocks=max_gpu_num_blocks,
        gpu_memory_utilization=gpu_memory_utilization,
        max_num_seqs=max_num_seqs,
        max_num_batched_tokens=max_num_batched_tokens,
        max_chunk_size=max_chunk_size,
        use_graph=bool(use_cuda_graph),
        pipeline=pipeline,
        seed=seed,
    )
    runner = ModelRunner(model, config, load_format=load_format, overrides=hf_overrides, device=device)
    model_dir = None if isinstance(model, Mapping) else Path(model)
    if tokenizer is None and model_dir is not None:
        tokenizer = load_tokenizer(model_dir)
    elif isinstance(tokenizer, (str, Path)):
        tokenizer = load_tokenizer(tokenizer)
    stop = load_stop_token_ids(model_dir, getattr(runner.config, "eos_token_ids", ()), tokenizer)
    scheduler = Scheduler(GpuExecutor(runner, Sampler(runner.device)), config, stop, tokenizer)
    scheduler.runner = runner
    return scheduler


class LLM:
    def __init__(
        self,
        model,
        tokenizer=None,
        max_seq_len: int = 2048,
        max_gpu_num_blocks: int | None = None,
        device: str = "cuda",
        use_cuda_graph: bool | None = None,
        quantization: str | None = None,
        tensor_parallel_size: int = 1,
        data_parallel_size: int = 1,
        kv_cache_dtype: str = "auto",
        hf_overrides: Mapping[str, Any] | None = None,
        *,
        dtype: str = "bfloat16",
        max_num_seqs: int = 32,
        max_num_batched_tokens: int = 8192,
        max_chunk_size: int = 512,
        page_size: int = 16,
        num_pages: int | None = None,
        load_format: str = "auto",
        seed: int = 0,
        pipeline: bool | None = None,
    ) -> None:
        if quantization is not None:
            raise ValueError("quantization is not supported by this engine (bfloat16 and float32 only)")
        if tensor_parallel_size != 1 or data_parallel_size != 1:
            raise ValueError("this engine runs on one GPU: parallel sizes must be 1")
        if kv_cache_dtype != "auto":
            raise ValueError("kv_cache_dtype must be 'auto': the cache has the engine's dtype")
        self.scheduler = build_engine(
            model, tokenizer=tokenizer, max_seq_len=max_seq_len, max_num_seqs=max_num_seqs,
            max_num_batched_tokens=max_num_batched_tokens, max_chunk_size=max_chunk_size,
            max_gpu_num_blocks=max_gpu_num_blocks, device=device,
            use_cuda_graph=True if use_cuda_graph is None else use_cuda_graph, dtype=dtype,
            page_size=page_size, num_pages=num_pages, load_format=load_format, seed=seed,
            hf_overrides=hf_overrides, pipeline=pipeline,
        )
        self.tokenizer = self.scheduler.tokenizer

    # ------------------------------------------------------------------ generation
    def _submit(self, prompts, sampling_params) -> list[Request]:
        if isinstance(prompts, str) or (prompts and isinstance(prompts[0], int)):
            prompts = [prompts]
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            params = [sampling_params or SamplingParams()] * len(prompts)
        else:
            params = list(sampling_params)
            if len(params) != len(prompts):
                raise ValueError(f"{len(params)} sampling_params for {len(prompts)} prompts")
        return [self.scheduler.add_request(p, sp) for p, sp in zip(prompts, params)]

    @staticmethod
    def _output(request: Request) -> RequestOutput:
        return RequestOutput(
            prompt=request.prompt,
            outputs=[
                CompletionOutput(
                    index=0,
                    text=request.text,
                    finish_reason=request.finish_reason,
                    token_ids=list(request.output_token_ids),
                    logprobs=list(request.output_logprobs) if request.output_logprobs is not None else None,
                )
            ],
            prompt_token_ids=list(request.prompt_token_ids),
            request_id=request.request_id,
            prompt_logprobs=list(request.prompt_logprobs) if request.prompt_logprobs is not None else None,
        )

    def generate(
        self,
        prompts: str | Sequence[int] | Sequence[str] | Sequence[Sequence[int]],
        sampling_params: SamplingParams | Sequence[SamplingParams] | None = None,
    ) -> list[RequestOutput]:
        """One :class:`RequestOutput` per prompt, in the order given
        (rapid_llm/engine/llm.py:150-195)."""
        requests = self._submit(prompts, sampling_params)
        self.scheduler.run_to_completion()
        return [self._output(r) for r in requests]

    def stream(self, prompts, sampling_params=None) -> Iterator[list[RequestOutput]]:
        """After every step, the outputs so far of the requests that advanced in it
        (rapid_llm/engine/llm.py:197-222)."""
        self._submit(prompts, sampling_params)
        while self.scheduler.has_unfinished_requests():
            advanced = self.scheduler.step()
            if advanced:
                yield [self._output(r) for r in advanced]
