"""Long decoding (one token a step up to the model's last position, across pages, key splits,
graph buckets and window trims) and the first tokens of a sequence, against the plain
implementation."""

import pytest
import torch

import parity
from plain_model import plain_forward, plain_load
from tiny_configs import TINY, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

F32_TOL = dict(rtol=2e-5, atol=3e-6)  # bfloat16: bounds relative to the logits' spread, see parity.py


def _close(got, want, dtype, label):
    if dtype == "float32":
        torch.testing.assert_close(got, want, **F32_TOL)
    else:
        parity.assert_bf16_close(got, want, label)


def _bucket(position, longest):
    """The context bound of the recorded step that serves a step whose largest position is
    ``position``: the next power of two from 512 on, within the engine's longest sequence."""
    bound = 512
    while bound <= position:
        bound *= 2
    return min(bound, longest)


def _runner(model_dir, dtype, page, max_seq_len, graph=False, num_pages=None, seqs=4):
    from rapid_llm_amd import EngineConfig, ModelRunner

    pages = num_pages or (seqs * (max_seq_len // page + 1) + 1)
    return ModelRunner(
        model_dir,
        EngineConfig(dtype=dtype, max_seq_len=max_seq_len, page_size=page, num_pages=pages,
                     max_num_seqs=seqs, use_graph=graph),
    )


@pytest.mark.parametrize("which", ["B", "C", "D", "F", "G", "H"])
@pytest.mark.parametrize("dtype,graph", [("float32", False), ("bfloat16", False), ("bfloat16", True)])
def test_long_decoding(tmp_path, which, dtype, graph):
    from rapid_llm_amd import StepEntry

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    pcfg, pw = plain_load(model_dir)
    limit = cfg["max_position_embeddings"]
    # two requests decode side by side, one from a 5-token prompt, one from a 70-token prompt
    toks = {"s": random_tokens(limit, cfg["vocab_size"], seed + 1), "l": random_tokens(limit - 40, cfg["vocab_size"], seed + 2)}
    want = {rid: plain_forward(pcfg, pw, t) for rid, t in toks.items()}
    runner = _runner(model_dir, dtype, page, limit, graph)
    got = {rid: [] for rid in toks}
    done = {"s": 5, "l": 70}
    for rid in toks:
        got[rid].append(runner.step([StepEntry(rid, toks[rid][: done[rid]], list(range(done[rid])))]).cpu())
    while any(done[r] < len(toks[r]) for r in toks):
        entries = [StepEntry(r, [toks[r][done[r]]], [0]) for r in toks if done[r] < len(toks[r])]
        logits = runner.step(entries).cpu()
        for k, e in enumerate(entries):
            got[e.request_id].append(logits[k : k + 1])
            done[e.request_id] += 1
    for rid in toks:
        out = torch.cat(got[rid])
        assert torch.isfinite(out).all()
        _close(out, want[rid], dtype, f"long/{which}/{'graph' if graph else 'eager'}/{rid}")
        runner.finish(rid)
    if graph:
        # two rows side by side from position 70 on, then the short request's row alone; every
        # context bucket those positions cross was recorded, and no other
        assert {key[0] for key in runner._graphs} == {1, 2}
        assert {key[1] for key in runner._graphs} == {_bucket(p, limit) for p in range(70, limit)}
    if which in ("C", "D"):  # windowed layers gave pages back while decoding
        assert runner.cache.num_free_pages(1) == runner.cache.pools[1].num_usable
    runner.cache.check_invariants()


def test_decoding_across_three_context_buckets(tmp_path):
    """One request decodes from position 400 to 1,099 from graphs: the recordings for contexts
    of up to 512, up to 1,024 and up to the engine's longest sequence follow each other, each
    with its own layout of the key splits, and every token's logits are the plain ones."""
    from rapid_llm_amd import StepEntry
    from rapid_llm_amd.weights import write_random_model

    cfg, page, seed = TINY["B"]
    limit = 1100
    model_dir = tmp_path / "long_b"
    write_random_model(dict(cfg, max_position_embeddings=limit), seed, model_dir, dtype="bfloat16", norm_std=0.1)
    pcfg, pw = plain_load(model_dir)
    toks = random_tokens(limit, cfg["vocab_size"], seed + 5)
    want = plain_forward(pcfg, pw, toks)
    runner = _runner(model_dir, "bfloat16", page, limit, graph=True, seqs=1)
    got = [runner.step([StepEntry("r", toks[:400], [399])]).cpu()]
    for t in toks[400:]:
        got.append(runner.step([StepEntry("r", [t], [0])]).cpu())
    _close(torch.cat(got), want[399:], "bfloat16", "long/three buckets")
    assert set(runner._graphs) == {(1, 512), (1, 1024), (1, limit)}
    runner.finish("r")
    runner.cache.check_invariants()


@pytest.mark.parametrize("which", ["A", "B", "C", "D", "F", "G", "H"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens(tmp_path, which, dtype):
    """Positions 0, 1, 2: a one-token prompt, its first decoded tokens, a two-token prompt cut
    into 1 + 1, and four one-token prompts in one batch."""
    from rapid_llm_amd import StepEntry

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    pcfg, pw = plain_load(model_dir)
    runner = _runner(model_dir, dtype, page, 64)
    toks = random_tokens(4, cfg["vocab_size"], seed)
    want = plain_forward(pcfg, pw, toks)
    rows = [runner.step([StepEntry("a", toks[:1], [0])]).cpu()]
    for t in toks[1:]:
        rows.append(runner.step([StepEntry("a", [t], [0])]).cpu())
    _close(torch.cat(rows), want, dtype, f"first/{which}/one by one")
    first = runner.step([StepEntry("b", toks[:1], [0])]).cpu()
    second = runner.step([StepEntry("b", toks[1:2], [0])]).cpu()
    _close(torch.cat([first, second]), want[:2], dtype, f"first/{which}/1+1")
    runner.finish("a")
    runner.finish("b")
    singles = random_tokens(4, cfg["vocab_size"], seed + 9)
    batch = runner.step([StepEntry(f"s{i}", [t], [0]) for i, t in enumerate(singles)]).cpu()
    _close(batch, torch.cat([plain_forward(pcfg, pw, [t]) for t in singles]), dtype, f"first/{which}/batch of 4")
    for i in range(len(singles)):
        runner.finish(f"s{i}")
    runner.cache.check_invariants()
