"""Trace replay: feed given token ids through the model step by step and write logits.

Nothing is sampled.  The replay drives the same :class:`ModelRunner` (model, step
function, cache manager, kernels) that generation uses; it has no forward pass, cache or
loader of its own.  The reference has no such tool; its nearest relative feeds given tokens
through an extend pass with ``return_logits=True`` when verifying speculated tokens
(rapid_llm/engine/scheduler.py:1076-1093).

Input, one JSON object per line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``<out>/<step>.f32`` holds the logits at the
wanted places in the order of the entries and of ``want``, little-endian float32
``[wanted, vocab]``.  After every step a line ``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import json
import sys
from pathlib import Path
from typing import IO, Iterable

import numpy as np

from ..config.engine_config import EngineConfig
from ..config.model_config import read_config_json
from .step import ModelRunner, StepEntry

REPLAY_PAGE_SIZE = 16
REPLAY_MAX_LIVE = 8  # traces keep up to four requests live; slots are cheap


def build_replay_runner(model_dir: str | Path, dtype: str, max_tokens: int) -> ModelRunner:
    """A runner whose page pool holds exactly ``max_tokens`` positions (rounded up to whole
    pages), so that a trace sized to it makes pages be used again."""
    body = read_config_json(model_dir)
    page = REPLAY_PAGE_SIZE
    pages = -(-int(max_tokens) // page)
    limit = int(body.get("max_position_embeddings", max_tokens))
    engine = EngineConfig(
        dtype=dtype,
        max_seq_len=max(2, min(limit, pages * page)),
        page_size=page,
        num_pages=pages + 1,  # + the null page
        max_num_seqs=REPLAY_MAX_LIVE,
        max_num_batched_tokens=max(2, pages * page),
        use_graph=False,
    )
    return ModelRunner(model_dir, engine)


def run_trace(
    runner: ModelRunner, lines: Iterable[str], out_dir: str | Path, log: IO[str] = sys.stdout
) -> int:
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    steps = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step_id = record["step"]
        entries = [
            StepEntry(str(e["id"]), list(e["tokens"]), list(e.get("want", ())))
            for e in record.get("entries", ())
        ]
        logits = runner.step(entries)
        if logits.shape[0] > 0:
            data = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            np.ascontiguousarray(data).tofile(out_dir / f"{step_id}.f32")
        for request_id in record.get("end", ()):
            runner.finish(str(request_id))
        print(f"done {step_id}", file=log, flush=True)
        steps += 1
    return steps
