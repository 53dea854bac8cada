"""The same requests cut into steps in every way, float32 and bfloat16, against the plain
implementation: whole; most in one step and the last 32 tokens one by one; portions of
changing size down to two tokens; mixed, up to four live with so few pages that they are
used again.  Pages are poisoned with NaN beforehand, so a read of a stale or unwritten row
cannot pass."""

import pytest
import torch

import parity
import replay_util as ru
from plain_model import plain_forward, plain_load
from tiny_configs import TINY, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

# float32: the engine and the plain implementation differ only in summation order
F32_TOL = dict(rtol=2e-5, atol=3e-6)
# bfloat16: bounds relative to the spread of the logits, see parity.py

LENGTHS = {
    "A": [13, 17, 25, 41, 70, 100],          # prompts 1/5/13/29 + 12 decoded, and two longer
    "B": [22, 37, 51, 84, 110, 170],         # prompts 2/17/31/64/90/150 + 20 decoded
    "C": [9, 33, 48, 77, 130, 201],
    "D": [12, 40, 66, 150, 333, 600],
    "E": [20, 35, 49, 64, 90, 200],          # portions of 17 to 64 tokens take the mid-size product
    "F": [3, 31, 33, 64, 97, 180],           # page of 32: requests within one page, at its edge, across several
    "G": [6, 21, 38, 75, 120, 190],          # head size 24; the window of 37 passes whole pages of 4
    "H": [5, 30, 65, 129, 260, 520],         # head size 128: tiles of 64 keys at, around and well beyond one and the window of 70
}


def _requests(which):
    cfg, _page, seed = TINY[which]
    return {f"q{i}": random_tokens(n, cfg["vocab_size"], seed * 100 + i) for i, n in enumerate(LENGTHS[which])}


_PLAIN = {}


def _plain(which, model_dir):
    key = (which, model_dir.name)
    if key not in _PLAIN:
        cfg, w = plain_load(model_dir)
        _PLAIN[key] = {rid: plain_forward(cfg, w, toks) for rid, toks in _requests(which).items()}
    return _PLAIN[key]


def _runner(model_dir, dtype, page, num_pages, max_seq_len):
    from rapid_llm_amd import EngineConfig, ModelRunner

    runner = ModelRunner(
        model_dir,
        EngineConfig(dtype=dtype, max_seq_len=max_seq_len, page_size=page, num_pages=num_pages,
                     max_num_seqs=4, use_graph=False),
    )
    for layer in runner.device_cache.layers:  # whatever is read before it is written shows
        if layer.owns_pages:
            layer.k.fill_(float("nan"))
            layer.v.fill_(float("nan"))
    return runner


def _check(got, want, dtype, label):
    if dtype != "float32":
        # all requests as one block: one spread, the worst row of any of them
        order = sorted(want)
        parity.assert_bf16_close(torch.cat([got[r] for r in order]), torch.cat([want[r] for r in order]), label)
        return
    tol = F32_TOL
    for rid in want:
        assert got[rid].shape == want[rid].shape, (label, rid)
        assert torch.isfinite(got[rid]).all(), (label, rid)
        try:
            torch.testing.assert_close(got[rid], want[rid], **tol)
        except AssertionError as exc:
            bad = ((got[rid] - want[rid]).abs() > tol["atol"] + tol["rtol"] * want[rid].abs()).any(dim=1)
            first = int(torch.nonzero(bad)[0])
            raise AssertionError(f"{label}: request {rid}, first wrong position {first}: {exc}") from None


@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E", "F", "G", "H"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_matches_plain(tmp_path, which, dtype):
    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    requests = _requests(which)
    want = _plain(which, model_dir)
    max_len = cfg["max_position_embeddings"]

    schedules = {
        "whole": ru.whole(requests),
        "decode32": ru.prefill_then_decode(requests, 32),
        "portions": ru.changing_portions(requests),
        "mixed": ru.mixed(requests, seed, max_tokens=None),
        "mixed_tight": ru.mixed(requests, seed + 1, max_tokens=2 * 64 * ((max(LENGTHS[which]) + 63) // 64)),
    }
    first = None
    for label, steps in schedules.items():
        pages = ru.pages_for(steps, requests, page)
        if label == "mixed":
            pages += 3
        runner = _runner(model_dir, dtype, page, pages + 1, max_len)
        got = ru.run_in_process(runner, steps)
        _check(got, want, dtype, f"{which}/{dtype}/{label}")
        runner.cache.check_invariants()
        assert not runner.cache.live_requests()
        for g in runner.cache.groups:
            assert runner.cache.pools[g.group_id].num_free == pages
        if dtype == "float32":
            err = max(ru.worst(got[r], want[r]) for r in want)
            print(f"{which}/{label}: worst float32 error {err:.3e}")
            # the float32 kernels sum in an order that depends on the position alone, so
            # cutting and batching change nothing at all
            if first is None:
                first = got
            for r in want:
                assert torch.equal(got[r], first[r]), f"{label}: {r} differs from the whole run"
        del runner


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, dtype):
    """The program itself, as a child process: mixed trace on the tight pool."""
    which = "B"
    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    requests = _requests(which)
    want = _plain(which, model_dir)
    max_tokens = 2 * 64 * ((max(LENGTHS[which]) + 63) // 64)
    steps = ru.mixed(requests, seed + 5, max_tokens=max_tokens)
    got = ru.run_trace_program(model_dir, dtype, steps, tmp_path / "out", max_tokens, cfg["vocab_size"])
    _check(got, want, dtype, f"trace_run/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_id_is_used_again_after_it_ended(tmp_path, dtype):
    """An id that ended names a new request the next time it appears: nothing of the old one
    (its length, its pages, its place in the block table) is left, also when the new one
    starts in the very step after and beside other requests."""
    which = "B"
    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    pcfg, pw = plain_load(model_dir)
    vocab = cfg["vocab_size"]
    first, second, other = (random_tokens(n, vocab, seed + n) for n in (45, 30, 38))
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": first[:40], "want": list(range(40))},
                                {"id": "o", "tokens": other[:20], "want": list(range(20))}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": first[40:], "want": list(range(5))},
                                {"id": "o", "tokens": other[20:21], "want": [0]}], "end": ["a"]},
        {"step": 2, "entries": [{"id": "a", "tokens": second[:7], "want": list(range(7))},
                                {"id": "o", "tokens": other[21:], "want": list(range(17))}], "end": ["o"]},
        {"step": 3, "entries": [{"id": "a", "tokens": second[7:], "want": list(range(23))}], "end": ["a"]},
    ]
    runner = _runner(model_dir, dtype, page, 7, cfg["max_position_embeddings"])  # 6 pages of 16: reuse
    rows = {"a1": [], "a2": [], "o": []}
    from rapid_llm_amd import StepEntry

    for step in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in step["entries"]]).cpu()
        at = 0
        for e in step["entries"]:
            key = "o" if e["id"] == "o" else ("a1" if step["step"] < 2 else "a2")
            rows[key].append(logits[at : at + len(e["want"])])
            at += len(e["want"])
        for rid in step["end"]:
            runner.finish(rid)
    want = {"a1": plain_forward(pcfg, pw, first), "a2": plain_forward(pcfg, pw, second), "o": plain_forward(pcfg, pw, other)}
    _check({k: torch.cat(v) for k, v in rows.items()}, want, dtype, f"id reuse/{dtype}")
    assert not runner.cache.live_requests()
    runner.cache.check_invariants()
