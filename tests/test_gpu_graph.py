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


@pytest.mark.parametrize("which", ["A", "C", "D", "F", "H"])
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


@pytest.mark.parametrize("which,batch", [("B", 17), ("B", 40), ("E", 23), ("E", 64), ("E", 100), ("E", 150)])
def test_graph_of_a_batch_beyond_the_skinny_product(tmp_path, which, batch):
    """More than 16 rows: the bfloat16 products are the library's, and in configuration E the
    output and down projections run as runs of K that the norms add (up to 192 rows, beyond 64 in
    blocks of 64 rows: the batches of 100 and 150 are recorded at 128 and 192 rows).  The graph replays are
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


# four kv heads of 64 channels: the fused decode kernel, and many workgroups from few requests
MANY_HEADS = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=72, num_attention_heads=8, num_key_value_heads=4,
    head_dim=64, intermediate_size=152, vocab_size=307, rope_theta=60000.0,
    rms_norm_eps=2e-6, tie_word_embeddings=True, max_position_embeddings=64,
    hidden_act="silu", attention_bias=False,
)


def test_graph_of_more_requests_than_the_chip_holds_workgroups(tmp_path):
    """200 requests on 4 kv heads are 800 decode workgroups, more than run at a time: the
    decode attention then takes the requests longest first, from an order that a kernel of the
    recorded step makes from the step's positions.  Between replays requests leave and others
    of other lengths take rows of the batch, so that a replay which kept the recording's
    order, or its lengths, would read other requests' keys or stop short of a request's own."""
    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry, write_random_model
    from rapid_llm_amd.kernels import ops

    batch, page, seed = 200, 8, 91
    assert batch * MANY_HEADS["num_key_value_heads"] > ops.chip().decode_resident
    model_dir = tmp_path / "many_heads"
    write_random_model(dict(MANY_HEADS), seed, model_dir, dtype="bfloat16", norm_std=0.1)
    make = lambda graph: ModelRunner(
        model_dir,
        EngineConfig(dtype="bfloat16", max_seq_len=64, page_size=page, num_pages=batch * (64 // page + 1) + 8,
                     max_num_seqs=batch + 1, use_graph=graph),
    )
    eager, graph = make(False), make(True)
    pcfg, pw = plain_load(model_dir)
    vocab = MANY_HEADS["vocab_size"]
    nxt, seqs = {}, {}

    def admit(rid, length, s):
        prompt = random_tokens(length, vocab, s)
        a = eager.step([StepEntry(rid, prompt, [length - 1])]).clone()
        graph.step([StepEntry(rid, prompt, [length - 1])])
        nxt[rid] = int(a[0].argmax())
        seqs[rid] = list(prompt)

    for i in range(batch):
        admit(f"m{i}", 2 + (i * 7) % 47, seed + i)
    for step in range(8):
        entries = [StepEntry(rid, [tok], [0]) for rid, tok in nxt.items()]
        a = eager.step(entries).clone()
        b = graph.step(entries).clone()
        torch.cuda.synchronize()
        for rid, tok in nxt.items():
            seqs[rid].append(tok)
        rids = list(nxt)
        parity.assert_bf16_close(b.cpu(), a.cpu(), f"graph of {batch} rows against eager/step {step}")
        if step in (0, 4, 7):  # against the plain implementation: the shortest, the longest, some between
            by_len = sorted(range(batch), key=lambda k: len(seqs[rids[k]]))
            rows = by_len[:3] + by_len[-3:] + by_len[batch // 2 :: 37]
            want = torch.stack([plain_forward(pcfg, pw, seqs[rids[k]])[-1] for k in rows])
            parity.assert_bf16_close(b.cpu()[rows], want, f"graph of {batch} rows/step {step}")
        for k, rid in enumerate(rids):
            nxt[rid] = int(a[k].argmax())
        if step == 3:  # twenty leave, twenty of other lengths arrive: the rows' lengths change
            for i in range(0, batch, 10):
                for r in (eager, graph):
                    r.finish(f"m{i}")
                del nxt[f"m{i}"], seqs[f"m{i}"]
            for j in range(batch // 10):
                admit(f"n{j}", 50 - (j * 11) % 49, seed + 1000 + j)
    assert any(key[0] >= batch for key in graph._graphs)
    for r in (eager, graph):
        for rid in nxt:
            r.finish(rid)
        r.cache.check_invariants()


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
