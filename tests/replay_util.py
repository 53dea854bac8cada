"""Ways of cutting the same requests into steps, and helpers to run them and compare.

A *trace* is a list of steps ``{"step", "entries": [{"id", "tokens", "want"}], "end"}`` in
the format ``bin/trace_run`` reads.  Every schedule asks for the logits at every position,
so any two schedules of the same requests can be compared position by position, and each
with the plain implementation.
"""

from __future__ import annotations

import json
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent


def whole(requests: dict[str, list[int]]) -> list[dict]:
    """Each request alone, whole, in one step."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append(
            {"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
        )
    return steps


def prefill_then_decode(requests: dict[str, list[int]], tail: int = 32) -> list[dict]:
    """Most of it in one step, then the last ``tail`` tokens one by one."""
    steps = []
    n = 0
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        cuts = [(0, head)] + [(i, i + 1) for i in range(head, len(toks))]
        for a, b in cuts:
            end = [rid] if b == len(toks) else []
            steps.append(
                {"step": n, "entries": [{"id": rid, "tokens": toks[a:b], "want": list(range(b - a))}], "end": end}
            )
            n += 1
    return steps


def changing_portions(requests: dict[str, list[int]], sizes=(7, 3, 2, 11, 2, 5, 17, 2, 4, 29)) -> list[dict]:
    """Portions of changing size, down to two tokens; one request at a time."""
    steps = []
    n = 0
    k = 0
    for rid, toks in requests.items():
        a = 0
        while a < len(toks):
            size = sizes[k % len(sizes)]
            k += 1
            b = min(len(toks), a + size)
            if len(toks) - b == 1:  # never leave a single token for a "portion"
                b = len(toks)
            end = [rid] if b == len(toks) else []
            steps.append(
                {"step": n, "entries": [{"id": rid, "tokens": toks[a:b], "want": list(range(b - a))}], "end": end}
            )
            n += 1
            a = b
    return steps


def mixed(
    requests: dict[str, list[int]],
    seed: int,
    max_live: int = 4,
    tail: int = 32,
    max_tokens: int | None = None,
    round_to: int = 64,
) -> list[dict]:
    """Up to ``max_live`` requests live at a time: portions of some beside single decoded
    tokens of others in one step, requests now and then left out of a step, new ones
    admitted as others end.  With ``max_tokens`` a request is only admitted when the live
    ones' final lengths (each rounded up to ``round_to``) still fit, so a small pool makes
    pages be used again."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: dict[str, dict] = {}
    steps = []
    n = 0

    def footprint(extra: int = 0) -> int:
        total = sum(-(-len(s["toks"]) // round_to) * round_to for s in live.values())
        return total + (-(-extra // round_to) * round_to if extra else 0)

    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting[0]
            if max_tokens is not None and footprint(len(toks)) > max_tokens:
                break
            waiting.pop(0)
            live[rid] = {"toks": toks, "done": 0, "decode_from": max(1, len(toks) - tail)}
        entries, end = [], []
        for rid, st in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue  # left out of this step, goes on later
            toks, a = st["toks"], st["done"]
            if a >= st["decode_from"]:
                b = a + 1
            else:
                size = rng.choice((2, 2, 3, 5, 8, 13, 24, 40))
                b = min(st["decode_from"], a + size)
                if st["decode_from"] - b == 1:
                    b = st["decode_from"]
            entries.append({"id": rid, "tokens": toks[a:b], "want": list(range(b - a))})
            st["done"] = b
            if b == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": n, "entries": entries, "end": end})
            n += 1
    return steps


def run_in_process(runner, steps: list[dict]) -> dict[str, torch.Tensor]:
    """Drive ``ModelRunner.step`` with a trace; returns per request ``[T, V]`` logits."""
    from rapid_llm_amd import StepEntry

    rows: dict[str, list[torch.Tensor]] = {}
    for step in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in step["entries"]]
        logits = runner.step(entries).cpu()
        at = 0
        for e in step["entries"]:
            k = len(e["want"])
            rows.setdefault(e["id"], []).append(logits[at : at + k])
            at += k
        assert at == logits.shape[0]
        for rid in step["end"]:
            runner.finish(rid)
    return {rid: torch.cat(parts) for rid, parts in rows.items()}


def run_trace_program(model_dir, dtype: str, steps: list[dict], out_dir, max_tokens: int, vocab: int,
                      timeout: int = 300) -> dict[str, torch.Tensor]:
    """Drive ``bin/trace_run`` as a child process, one step after each ``done`` line."""
    proc = subprocess.Popen(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
         "--out", str(out_dir), "--max-tokens", str(max_tokens)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1,
    )
    try:
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {step['step']}", f"unexpected reply {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=timeout) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    rows: dict[str, list[torch.Tensor]] = {}
    for step in steps:
        wanted = sum(len(e["want"]) for e in step["entries"])
        path = Path(out_dir) / f"{step['step']}.f32"
        if wanted == 0:
            assert not path.exists()
            continue
        data = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab).copy())
        at = 0
        for e in step["entries"]:
            k = len(e["want"])
            rows.setdefault(e["id"], []).append(data[at : at + k])
            at += k
    return {rid: torch.cat(parts) for rid, parts in rows.items()}


def pages_for(steps: list[dict], requests: dict[str, list[int]], page: int) -> int:
    """Fewest pages (without the null page) under which the trace still fits: the peak,
    over steps, of the live requests' pages after the step's tokens are in."""
    held: dict[str, int] = {}
    peak = 0
    for step in steps:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // page) for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return peak


def worst(got: torch.Tensor, want: torch.Tensor) -> float:
    return float((got.double() - want.double()).abs().max())
