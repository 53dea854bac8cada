"""Where a run's device time goes, part by part: HIP events around every part's ``forward``.

Events, not host clocks, because a launch returns long before its kernels have run; the
reference records its regions the same way (rapid_llm/batch_overlap/overlap.py:247-314,
``Timeline.region`` / ``collect`` / ``summary``).  Recording costs two events a region, so it
is switched on only for the runs that are to be looked at (``rapid-llm bench --profile``),
and those run every step eagerly: a recorded step is one graph launch and has no regions.

What a region holds is what the part launched, not what the part is named for: a product
that the norm after it absorbs (``parts/lazy.py``) is timed with that norm.
"""

from __future__ import annotations

from collections import defaultdict
from contextlib import contextmanager
from dataclasses import dataclass, field
from typing import Iterator

import torch


@dataclass
class RegionRecord:
    phase: str
    name: str
    ms: float


@dataclass
class Timeline:
    enabled: bool = True
    phase: str = ""  # what kind of step is running; set by whoever drives the steps
    _pending: list[tuple[str, str, torch.cuda.Event, torch.cuda.Event]] = field(default_factory=list, repr=False)

    @contextmanager
    def region(self, name: str) -> Iterator[None]:
        """Time what is queued on the current stream inside the block; free when disabled."""
        if not self.enabled:
            yield
            return
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        try:
            yield
        finally:
            end.record()
            self._pending.append((self.phase, name, start, end))

    def collect(self) -> list[RegionRecord]:
        """Wait for every recorded region and return them in the order they were opened."""
        records = []
        for phase, name, start, end in self._pending:
            end.synchronize()
            records.append(RegionRecord(phase, name, start.elapsed_time(end)))
        self._pending.clear()
        return records

    def summary(self) -> str:
        """A table per phase: region, calls, total milliseconds, share of the phase."""
        by_phase: dict[str, dict[str, list[float]]] = defaultdict(lambda: defaultdict(list))
        for r in self.collect():
            by_phase[r.phase][r.name].append(r.ms)
        lines = []
        for phase, regions in by_phase.items():
            total = sum(sum(v) for v in regions.values()) or 1.0
            lines.append(f"{phase or 'steps'}: {total:.3f} ms inside parts")
            for name, times in sorted(regions.items(), key=lambda kv: -sum(kv[1])):
                lines.append(
                    f"  {name:<28} {len(times):>7} calls {sum(times):>10.3f} ms {100 * sum(times) / total:>5.1f}%"
                    f" {1e3 * sum(times) / len(times):>9.1f} us/call"
                )
        return "\n".join(lines)


def instrument(runner, timeline: Timeline) -> None:
    """Put a region around every part of ``runner``'s model (named after the part's role and
    class) and make every step say whether it holds portions of prompts or single tokens only.
    The parts' own classes are untouched: the wrappers sit on the instances."""
    model = runner.model

    def wrap(part, role: str) -> None:
        inner = part.forward
        name = f"{role} ({type(part).__name__})"

        def timed(*args, **kwargs):
            with timeline.region(name):
                return inner(*args, **kwargs)

        part.forward = timed

    wrap(model.embed, "embedding")
    wrap(model.final_norm, "final norm")
    wrap(model.output, "output projection")
    for block in model.blocks:
        # a block that names its parts this way is timed part by part, any other as a whole
        named = [(role, getattr(block, attr, None)) for role, attr in (
            ("mixer norm", "mixer_norm"), ("mixer", "mixer"),
            ("feed-forward norm", "feed_forward_norm"), ("feed-forward", "feed_forward"))]
        if all(part is not None for _, part in named):
            for role, part in named:
                wrap(part, role)
        else:
            wrap(block, "block")

    step = runner.step

    def phased(entries, use_graph=None):
        timeline.phase = "decode steps" if all(len(e.tokens) == 1 for e in entries) else "steps with prompt portions"
        return step(entries, use_graph=False)  # a replayed graph has no regions

    runner.step = phased
