"""Run-time knobs of the engine, apart from the model's own configuration.

Names follow the reference where it has them: ``max_seq_len``, ``max_num_seqs``,
``max_num_batched_tokens``, ``max_chunk_size`` (rapid_llm/engine/batch_planner.py:151-153,
:202-240) and ``max_gpu_num_blocks``, the cache capacity in tokens (README.md:121).
"""

from __future__ import annotations

from dataclasses import dataclass

from .model_config import ConfigError, normalise_dtype_name


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"  # "bfloat16" | "float32"
    max_seq_len: int = 2048  # longest sequence one request may reach
    page_size: int = 16  # tokens in a cache page (rapid_llm/engine/prefix_cache.py:32)
    num_pages: int | None = None  # pages per cache group; None: from max_gpu_num_blocks / memory
    max_gpu_num_blocks: int | None = None  # cache capacity in tokens, the reference's knob
    gpu_memory_utilization: float = 0.9  # rapid_llm/executor/kv_cache_manager.py:91-130
    max_num_seqs: int = 32
    max_num_batched_tokens: int = 8192
    max_chunk_size: int = 512  # 0 turns chunked prefill off
    use_graph: bool = True  # replay decode-only steps from a captured HIP graph
    # what to do with a decode step whose recording would hold a product of the library (a step
    # of more rows than this package's own products take, or a matrix whose sizes they refuse):
    # "record" it as it is, run such steps "eager"ly, or "refuse" with an error (tests)
    library_in_graph: str = "record"
    # queue the next step before the last one's tokens are read (rapid_llm/engine/scheduler.py:
    # 302-303); None: the environment variable RAPID_LLM_PIPELINE, on when it is not set
    pipeline: bool | None = None
    seed: int = 0

    def __post_init__(self) -> None:
        object.__setattr__(self, "dtype", normalise_dtype_name(self.dtype))
        # rapid_llm/engine/batch_planner.py:212-240
        if self.max_seq_len < 2:
            raise ConfigError(f"max_seq_len must be >= 2, got {self.max_seq_len}")
        if self.page_size < 4 or self.page_size % 4:
            raise ConfigError(
                f"page_size must be a positive multiple of 4, got {self.page_size} "
                "(the value cache is stored transposed in groups of four keys)"
            )
        for name in ("max_num_seqs", "max_num_batched_tokens"):
            if getattr(self, name) < 1:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.library_in_graph not in ("record", "eager", "refuse"):
            raise ConfigError(
                f"library_in_graph must be 'record', 'eager' or 'refuse', got {self.library_in_graph!r}"
            )
        if self.max_chunk_size < 0:
            raise ConfigError(f"max_chunk_size must be >= 0, got {self.max_chunk_size}")
        if self.max_chunk_size == 0 and self.max_num_batched_tokens < self.max_seq_len:
            raise ConfigError(
                "with chunked prefill off (max_chunk_size=0) max_num_batched_tokens "
                f"({self.max_num_batched_tokens}) must cover max_seq_len ({self.max_seq_len})"
            )
        if self.num_pages is not None and self.num_pages < 2:
            raise ConfigError("num_pages must be >= 2 (page 0 is the null page)")
        if not 0.0 < self.gpu_memory_utilization <= 1.0:
            raise ConfigError("gpu_memory_utilization must be in (0, 1]")
