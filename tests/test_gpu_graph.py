"""Decode steps replayed from a captured HIP graph give what eager steps give: every replay
is checked, with eager prompt steps, admissions and synchronisations between replays."""

import pytest
import torch

import parity
from plain_model import plain_forward, plain_load
from tiny_configs import TINY, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu


def _runner(model_dir, dtype, page, graph):
    from rapid_llm_amd import EngineConfig, ModelRunner

    return ModelRunner(
        model_dir,
        EngineConfig(dtype=dtype, max_seq_len=128, page_size=page, num_pages=80, max_num_seqs=4, use_graph=graph),
    )


@pytest.mark.parametrize("which", ["A", "C", "D", "F"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_match_eager(tmp_path, which, dtype):
    from rapid_llm_amd import StepEntry

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    eager = _runner(model_dir, dtype, page, graph=False)
    graph = _runner(model_dir, dtype, page, graph=True)
    vocab = cfg["vocab_size"]
    prompts = {f"g{i}": random_tokens(n, vocab, seed + i) for i, n in enumerate([9, 30, 3])}
    pairs = []

    def both(entries):
        a = eager.step(entries).clone()
        b = graph.step(entries).clone()
        torch.cuda.synchronize()
        if dtype == "float32":
            assert torch.equal(a, b)  # same kernels, same order of sums
        else:
            # a recorded step lays the key splits out for its bucket's longest context: other sums
            pairs.append((a.cpu(), b.cpu()))
        return a

    nxt = {}
    live = []
    for rid in ("g0", "g1"):
        logits = both([StepEntry(rid, prompts[rid], [len(prompts[rid]) - 1])])
        nxt[rid] = int(logits[0].argmax())
        live.append(rid)
    for step in range(40):
        logits = both([StepEntry(rid, [nxt[rid]], [0]) for rid in live])
        for k, rid in enumerate(live):
            nxt[rid] = int(logits[k].argmax())
        if step == 10:  # a new request arrives: an eager prompt step, then a larger batch
            logits = both([StepEntry("g2", prompts["g2"], [2])])
            nxt["g2"] = int(logits[0].argmax())
            live.append("g2")
        if step == 25:  # one leaves: back to a batch size whose graph exists already
            eager.finish("g0")
            graph.finish("g0")
            live.remove("g0")
    assert graph._graphs, "no graph was captured"
    if pairs:
        parity.assert_bf16_close(torch.cat([b for _, b in pairs]), torch.cat([a for a, _ in pairs]),
                                 f"graph against eager/{which}")
    for r in (eager, graph):
        for rid in live:
            r.finish(rid)
        r.cache.check_invariants()


@pytest.mark.parametrize("which,batch", [("B", 17), ("B", 40), ("E", 23), ("E", 64)])
def test_graph_of_a_batch_beyond_the_skinny_product(tmp_path, which, batch):
    """More than 16 rows: the bfloat16 products are the library's, and in configuration E the
    output and down projections run as runs of K that the norms add.  The graph replays are
    checked one by one against eager steps of a second engine, with eager work between."""
    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, "bfloat16")
    make = lambda graph: ModelRunner(
        model_dir,
        EngineConfig(dtype="bfloat16", max_seq_len=64, page_size=page, num_pages=batch * 4 + 8,
                     max_num_seqs=batch + 1, use_graph=graph),
    )
    eager, graph = make(False), make(True)
    pcfg, pw = plain_load(model_dir)
    vocab = cfg["vocab_size"]
    nxt, seqs = {}, {}
    for i in range(batch):
        prompt = random_tokens(3 + i % 9, vocab, seed + i)
        a = eager.step([StepEntry(f"b{i}", prompt, [len(prompt) - 1])]).clone()
        b = graph.step([StepEntry(f"b{i}", prompt, [len(prompt) - 1])]).clone()
        assert torch.equal(a, b)  # a prompt's step is never recorded: the same kernels ran
        nxt[f"b{i}"] = int(a[0].argmax())
        seqs[f"b{i}"] = list(prompt)
    for step in range(12):
        entries = [StepEntry(rid, [tok], [0]) for rid, tok in nxt.items()]
        a = eager.step(entries).clone()
        b = graph.step(entries).clone()
        torch.cuda.synchronize()
        for rid, tok in nxt.items():
            seqs[rid].append(tok)
        if step in (0, 5, 11):  # replays against the plain implementation, not only against eager
            want = torch.stack([plain_forward(pcfg, pw, seqs[rid])[-1] for rid in nxt])
            parity.assert_bf16_close(b.cpu(), want, f"graph of {batch} rows/{which}/step {step}")
        parity.assert_bf16_close(b.cpu(), a.cpu(), f"graph of {batch} rows against eager/{which}/step {step}")
        if step % 4 == 1:  # eager work of the program's own between replays
            extra = random_tokens(5, vocab, step)
            graph.step([StepEntry("x", extra, [4])])
            graph.finish("x")
            eager.step([StepEntry("x", extra, [4])])
            eager.finish("x")
        for k, rid in enumerate(nxt):
            nxt[rid] = int(a[k].argmax())
    assert any(key[0] >= batch for key in graph._graphs)  # padded up to a size of the ladder


def test_ragged_batches_share_a_few_graphs(tmp_path):
    """Requests that end at different times walk the batch size down one by one: the steps are
    padded with filler rows to a ladder of sizes, so few graphs are captured; with and without
    graphs every token lies within rounding of the plain implementation's choice."""
    from rapid_llm_amd import LLM, SamplingParams

    cfg, page, seed = TINY["D"]
    model_dir = make_model_dir(tmp_path, "D", "bfloat16")
    prompts = [random_tokens(3 + i, cfg["vocab_size"], seed + i) for i in range(11)]
    params = [SamplingParams(temperature=0.0, max_gen_len=4 + 3 * i) for i in range(11)]
    pcfg, pw = plain_load(model_dir)
    for graph in (False, True):
        llm = LLM(str(model_dir), dtype="bfloat16", max_seq_len=128, page_size=page, num_pages=200,
                  max_num_seqs=16, use_cuda_graph=graph)
        outs = [o.token_ids for o in llm.generate(prompts, params)]
        if graph:
            sizes = sorted({key[0] for key in llm.scheduler.runner._graphs})
            assert sizes and set(sizes) <= {1, 2, 4, 8, 12, 16}, sizes
        assert [len(o) for o in outs] == [4 + 3 * i for i in range(11)]
        # bfloat16: a near-tie may fall the other way, so the two engines' tokens need not agree;
        # each token must lie within rounding of the plain choice given the tokens before it
        for i, (prompt, out) in enumerate(zip(prompts, outs)):
            ids = list(prompt)
            for tok in out:
                parity.assert_near_choice(plain_forward(pcfg, pw, ids)[-1], tok, f"ragged/graph={graph}/request {i}")
                ids.append(tok)
