"""Two layers at the widths the benchmark runs (hidden 4,096, 32 query and 8 kv heads of 128,
intermediate 12,288, an untied vocabulary of 151,936), float32 and bfloat16, against the plain
implementation on the CPU: one 2,048-token step, portions of 512 behind a growing prefix, then
single tokens at batch 1, 8 and 64 replayed from graphs whose context bucket is 4,096.

At these widths run kernels and launch shapes that no tiny configuration reaches: the few-row
product with two tiles of weight rows a workgroup, the output projection over 151,936 rows,
the product for 17 to 64 rows inside a model, the fused decode kernel at head size 128 with
keys split for a bucket of 4,096, the prefill kernel with two wave groups on a tile and with
tiles cut into key runs.  The pattern is the reference's whole-model comparison
(tests/cpu/test_inference.py:108-126) at the benchmark's sizes."""

import pytest
import torch

import parity
from plain_model import plain_forward, plain_load
from tiny_configs import random_tokens

pytestmark = pytest.mark.gpu

CONFIG = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
    head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=4096,
    hidden_act="silu", attention_bias=False,
)
PAGE = 16
DECODE_STEPS = 2  # single-token steps at batch 1 and 8
# at batch 64: three replays, with an eager prompt step of another request between them, each
# checked against the plain implementation
BATCH64_STEPS = 3
# float32: sums of 4,096 to 12,288 terms in another order than the plain product's
F32_TOL = dict(rtol=1e-4, atol=5e-5)


class _Sequences:
    """The requests of the test: their tokens, and which positions' logits are compared."""

    def __init__(self):
        vocab = CONFIG["vocab_size"]
        tail = 2 * DECODE_STEPS + 1 + BATCH64_STEPS  # the longest-lived request decodes at batch 1 and 8, in the mixed step and at batch 64
        self.prompt = {"a": 2048, "b": 2560, "c": 700}
        for i in range(61):
            self.prompt[f"s{i}"] = 3 + (i * 7) % 90
        for i in range(BATCH64_STEPS):
            self.prompt[f"z{i}"] = 40 + 30 * i  # admitted between the replays at batch 64, never decoded
        self.tokens = {rid: random_tokens(n + tail, vocab, 1000 + k) for k, (rid, n) in enumerate(self.prompt.items())}
        self.rows: dict[str, list[int]] = {rid: [] for rid in self.prompt}

    def want(self, rid, positions):
        self.rows[rid].extend(positions)
        return list(positions)


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    from rapid_llm_amd import write_random_model

    folder = tmp_path_factory.mktemp("real_widths") / "two_layers"
    write_random_model(dict(CONFIG), 7, folder, dtype="bfloat16", norm_std=0.1)
    return folder


def _plan(seqs):
    """The steps of the test as (label, entries, graph) with entries (request, first position,
    count, wanted places); positions are filled in as the plan is laid out."""
    done = {rid: 0 for rid in seqs.prompt}
    steps = []

    def entry(rid, count, want):
        e = (rid, done[rid], count, want)
        seqs.want(rid, [done[rid] + w for w in want])
        done[rid] += count
        return e

    # one 2,048-token step: the prefill kernel's two-wave-group shape; every 64th row and the end
    steps.append(("a whole", [entry("a", 2048, list(range(0, 2048, 64)) + list(range(2040, 2048)))], False))
    for i in range(DECODE_STEPS):
        steps.append((f"batch 1 step {i}", [entry("a", 1, [0])], True))
    # portions of 512: from the second on, few long tiles whose keys are cut into runs
    for p in range(5):
        steps.append((f"b portion {p}", [entry("b", 512, [0, 1, 255, 256, 510, 511])], False))
    # six prompts in one step beside nothing else, then batch 8
    firsts = ["c"] + [f"s{i}" for i in range(5)]
    steps.append(("six prompts", [entry(r, seqs.prompt[r], [seqs.prompt[r] - 1]) for r in firsts], False))
    eight = ["a", "b"] + firsts
    for i in range(DECODE_STEPS):
        steps.append((f"batch 8 step {i}", [entry(r, 1, [0]) for r in eight], True))
    # 56 more prompts beside the eight's next tokens (portions beside decoded tokens), then batch 64
    rest = [f"s{i}" for i in range(5, 61)]
    steps.append(("mixed", [entry(r, 1, [0]) for r in eight] + [entry(r, seqs.prompt[r], [seqs.prompt[r] - 1]) for r in rest], False))
    everyone = eight + rest
    for i in range(BATCH64_STEPS):
        steps.append((f"batch 64 step {i}", [entry(r, 1, [0]) for r in everyone], True))
        z = f"z{i}"
        steps.append((f"a prompt between the replays ({z})", [entry(z, seqs.prompt[z], [seqs.prompt[z] - 1])], False))
    return steps


@pytest.fixture(scope="module")
def reference(model):
    """The plan and the plain implementation's logits at every compared position (the weights as
    the bfloat16 checkpoint stores them, arithmetic in float32: the oracle of both engines)."""
    seqs = _Sequences()
    steps = _plan(seqs)
    pcfg, pw = plain_load(model)
    plain = {}
    for rid, rows in seqs.rows.items():
        length = max(rows) + 1
        logits = plain_forward(pcfg, pw, seqs.tokens[rid][:length], rows=rows)
        plain[rid] = {pos: logits[i] for i, pos in enumerate(rows)}
    del pw
    return seqs, steps, plain


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_widths_match_plain(model, reference, dtype):
    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry

    seqs, steps, plain = reference
    runner = ModelRunner(
        model,
        # a recorded step of up to 64 rows holds this package's kernels only, or the engine raises
        EngineConfig(dtype=dtype, max_seq_len=4096, page_size=PAGE, num_pages=1200, max_num_seqs=68, use_graph=True,
                     library_in_graph="refuse"),
    )
    for label, entries, graph in steps:
        before = set(runner._graphs)
        logits = runner.step(
            [StepEntry(rid, seqs.tokens[rid][start : start + count], want) for rid, start, count, want in entries]
        ).cpu()
        want = torch.stack([plain[rid][start + w] for rid, start, count, ws in entries for w in ws])
        assert logits.shape == want.shape, label
        if graph:
            keys = set(runner._graphs)
            assert keys, f"{label}: the step was not replayed from a graph"
            bucket = {k for k in keys if k[0] >= len(entries) and k[1] == 4096}
            assert bucket, f"{label}: no graph for {len(entries)} rows in the bucket of 4,096 ({sorted(keys)})"
        else:
            assert set(runner._graphs) == before, f"{label}: a step with a portion was recorded"
        if dtype == "float32":
            err = float((logits - want).abs().max())
            print(f"real widths float32 {label}: worst error {err:.3e} (logits spread {float(want.std()):.3f})")
            torch.testing.assert_close(logits, want, **F32_TOL)
        else:
            parity.assert_bf16_close(logits, want, f"real widths/{label}")
    assert runner.graph_library_products and not any(runner.graph_library_products.values())
    for rid in seqs.prompt:
        runner.finish(rid)
    runner.cache.check_invariants()
    assert not runner.cache.live_requests()


def test_recorded_steps_of_up_to_64_rows_hold_no_library_product(model):
    """Every batch size of the ladder up to 64 at the benchmark's widths: the step is recorded
    under ``library_in_graph="refuse"`` (a product that went to the library would raise), replayed,
    and gives the plain implementation's logits.  Beyond 64 rows the wide products are the
    library's: such a step is recorded as it is by default, runs eagerly when the engine is
    told so, and is refused when it is told that."""
    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry
    from rapid_llm_amd.engine.step import GRAPH_BATCHES
    from rapid_llm_amd.kernels import ops

    pcfg, pw = plain_load(model)
    vocab = CONFIG["vocab_size"]
    tokens = random_tokens(96, vocab, 77)
    plain = {t: plain_forward(pcfg, pw, [t])[0] for t in sorted(set(tokens))}
    del pw
    common = dict(dtype="bfloat16", max_seq_len=4096, page_size=PAGE, num_pages=200, max_num_seqs=100, use_graph=True)
    runner = ModelRunner(model, EngineConfig(library_in_graph="refuse", **common))
    for rows in [b for b in GRAPH_BATCHES if b <= 64]:
        for rep in range(2):  # the recording's first replay, and a second with other tokens
            chosen = tokens[rep : rep + rows]
            logits = runner.step([StepEntry(f"r{i}", [t], [0]) for i, t in enumerate(chosen)]).cpu()
            parity.assert_bf16_close(logits, torch.stack([plain[t] for t in chosen]), f"ladder/{rows} rows/{rep}")
            for i in range(rows):
                runner.finish(f"r{i}")
        assert runner.graph_library_products[(rows, 512)] == 0
    ninety_six = [StepEntry(f"r{i}", [t], [0]) for i, t in enumerate(tokens)]
    with pytest.raises(ops.KernelError, match="96 rows would record"):
        runner.step(ninety_six)
    for i in range(96):
        runner.finish(f"r{i}")
    want = torch.stack([plain[t] for t in tokens])
    for policy in ("eager", "record"):
        other = ModelRunner(model, EngineConfig(library_in_graph=policy, **common))
        for rep in range(2):
            parity.assert_bf16_close(other.step(ninety_six).cpu(), want, f"ladder/96 rows/{policy}/{rep}")
            for i in range(96):
                other.finish(f"r{i}")
        assert ((96, 512) in other._graphs) == (policy == "record")
        assert other.graph_library_products[(96, 512)] > 0


# Two layers at the widths of the family's largest dense model (hidden 5,120, 64 query heads on 8
# kv heads of 128: groups of 8, intermediate 25,600) with the vocabulary cut to 32,000 so that
# the plain implementation's float32 copy stays within a few gigabytes, at a long context: a
# 9,000-token prompt in portions of 8,192 and 808 (the second a few long tiles behind a long
# prefix), then single tokens at batch 1, 8 and 32 replayed from graphs of the 16,384 bucket.
LARGE = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
    head_dim=128, intermediate_size=25600, vocab_size=32000, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=16384,
    hidden_act="silu", attention_bias=False,
)
# The same at the widths of the family's 14B model (40 query heads on 8 kv heads: groups of 5,
# which fill five sixteenths of the attention kernels' blocks of 16 rows; intermediate 17,408,
# whose gate/up matrix is 5.3 tiles a compute unit for the product for 17 to 64 rows), a
# 2,600-token prompt in portions of 2,048 and 552 and graphs of the 4,096 bucket.
GROUP5 = dict(LARGE, num_attention_heads=40, intermediate_size=17408, vocab_size=20000, max_position_embeddings=4096)
# name -> (configuration, prompt tokens, first portion, context bucket = max_seq_len, pages)
LARGE_CASES = {
    "largest": (LARGE, 9000, 8192, 16384, 800),
    "group5": (GROUP5, 2600, 2048, 4096, 400),
}
LARGE_STEPS = 2  # single-token steps at each batch size


def _large_plan(vocab, prompt_len, portion):
    """(tokens by request, steps as (label, [(request, start, count, wanted places)], graph))."""
    prompt = {"long": prompt_len}
    for i in range(31):
        prompt[f"s{i}"] = 2 + (i * 11) % 70
    tokens = {r: random_tokens(n + 3 * LARGE_STEPS, vocab, 2000 + k) for k, (r, n) in enumerate(prompt.items())}
    done = {r: 0 for r in prompt}
    steps = []

    def entry(rid, count, want):
        e = (rid, done[rid], count, want)
        done[rid] += count
        return e

    rest_len = prompt_len - portion
    steps.append(("first portion", [entry("long", portion, [0, 1, portion // 2 - 1, portion // 2, portion - 2, portion - 1])], False))
    steps.append(("second portion behind the first", [entry("long", rest_len, [0, 1, rest_len // 2, rest_len - 2, rest_len - 1])], False))
    for i in range(LARGE_STEPS):
        steps.append((f"batch 1 step {i}", [entry("long", 1, [0])], True))
    seven = [f"s{i}" for i in range(7)]
    steps.append(("seven prompts", [entry(r, prompt[r], [prompt[r] - 1]) for r in seven], False))
    for i in range(LARGE_STEPS):
        steps.append((f"batch 8 step {i}", [entry(r, 1, [0]) for r in ["long"] + seven], True))
    rest = [f"s{i}" for i in range(7, 31)]
    steps.append(("24 prompts", [entry(r, prompt[r], [prompt[r] - 1]) for r in rest], False))
    for i in range(LARGE_STEPS):
        steps.append((f"batch 32 step {i}", [entry(r, 1, [0]) for r in ["long"] + seven + rest], True))
    return tokens, steps


@pytest.fixture(scope="module", params=sorted(LARGE_CASES))
def large(request, tmp_path_factory):
    """The model folder, the plan and the plain logits at every compared position."""
    from rapid_llm_amd import write_random_model

    config, prompt_len, portion, bucket, pages = LARGE_CASES[request.param]
    folder = tmp_path_factory.mktemp(f"{request.param}_widths") / "two_layers"
    write_random_model(dict(config), 13, folder, dtype="bfloat16", norm_std=0.1)
    tokens, steps = _large_plan(config["vocab_size"], prompt_len, portion)
    rows: dict[str, list[int]] = {r: [] for r in tokens}
    for _label, entries, _graph in steps:
        for rid, start, _count, want in entries:
            rows[rid].extend(start + w for w in want)
    pcfg, pw = plain_load(folder)
    plain = {}
    for rid, at in rows.items():
        logits = plain_forward(pcfg, pw, tokens[rid][: max(at) + 1], rows=at)
        plain[rid] = {pos: logits[i] for i, pos in enumerate(at)}
    del pw
    return request.param, folder, tokens, steps, plain, bucket, pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_large_widths_at_a_long_context_match_plain(large, dtype):
    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry

    name, folder, tokens, steps, plain, bucket, pages = large
    runner = ModelRunner(
        folder,
        EngineConfig(dtype=dtype, max_seq_len=bucket, page_size=PAGE, num_pages=pages, max_num_seqs=32, use_graph=True),
    )
    for label, entries, graph in steps:
        before = set(runner._graphs)
        logits = runner.step(
            [StepEntry(rid, tokens[rid][start : start + count], want) for rid, start, count, want in entries]
        ).cpu()
        want = torch.stack([plain[rid][start + w] for rid, start, count, ws in entries for w in ws])
        assert logits.shape == want.shape, label
        if graph:
            assert (len(entries), bucket) in runner._graphs, f"{label}: no graph of the {bucket} bucket ({sorted(runner._graphs)})"
        else:
            assert set(runner._graphs) == before, f"{label}: a step with a portion was recorded"
        if dtype == "float32":
            err = float((logits - want).abs().max())
            print(f"{name} widths float32 {label}: worst error {err:.3e} (logits spread {float(want.std()):.3f})")
            torch.testing.assert_close(logits, want, **F32_TOL)
        else:
            parity.assert_bf16_close(logits, want, f"{name} widths/{label}")
    for rid in tokens:
        runner.finish(rid)
    runner.cache.check_invariants()


# Two layers at the widths of the family's smallest model (hidden 1,024, 16 query and 8 kv heads
# of 128, intermediate 3,072), a short vocabulary: its QKV and gate/up matrices are the few
# megabytes for which steps of 17 to 512 rows run the one-launch tile product (with SwiGLU in
# its epilogue) instead of the library's kernels, and 200 requests on 8 kv heads are more decode
# workgroups than run at once, so that the attention takes them longest first.
SMALL = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8,
    head_dim=128, intermediate_size=3072, vocab_size=1500, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=256,
    hidden_act="silu", attention_bias=False,
)


@pytest.mark.parametrize("graph", [False, True], ids=["eager", "graph"])
def test_smallest_widths_in_steps_of_tens_and_hundreds_of_rows(tmp_path, monkeypatch, graph):
    from rapid_llm_amd import EngineConfig, ModelRunner, StepEntry, write_random_model
    from rapid_llm_amd.kernels import ops

    folder = tmp_path / "small"
    write_random_model(dict(SMALL), 3, folder, dtype="bfloat16", norm_std=0.1)
    pcfg, pw = plain_load(folder)
    took = []
    applies = ops._tile_applies
    monkeypatch.setattr(ops, "_tile_applies", lambda *a: took.append(applies(*a)) or took[-1])
    runner = ModelRunner(
        folder, EngineConfig(dtype="bfloat16", max_seq_len=128, page_size=16, num_pages=200 * 8 + 8,
                             max_num_seqs=201, use_graph=graph),
    )
    vocab = SMALL["vocab_size"]
    seqs = {f"r{i}": random_tokens(2 + (i * 13) % 90, vocab, 500 + i) for i in range(200)}
    # prompts, several a step: 100 to 500 rows, mostly the tile product's sizes, some the library's
    rids = list(seqs)
    for at in range(0, 200, 8):
        runner.step([StepEntry(r, seqs[r], []) for r in rids[at : at + 8]])
    gen = torch.Generator().manual_seed(9)
    for live in (40, 200, 17, 130):  # single tokens: 17 to 256 rows
        chosen = [rids[int(i)] for i in torch.randperm(200, generator=gen)[:live]]
        tokens = {r: int(torch.randint(0, vocab, (1,), generator=gen)) for r in chosen}
        took.clear()
        logits = runner.step([StepEntry(r, [tokens[r]], [0]) for r in chosen]).cpu()
        assert any(took), f"{live} rows: the tile product was not used"
        for r in chosen:
            seqs[r].append(tokens[r])
        order = sorted(range(live), key=lambda i: len(seqs[chosen[i]]))
        rows = order[:4] + order[-4:] + order[live // 2 : live // 2 + 4]
        want = torch.stack([plain_forward(pcfg, pw, seqs[chosen[i]])[-1] for i in rows])
        parity.assert_bf16_close(logits[rows], want, f"smallest widths/{live} rows/graph={graph}")
    if graph:
        assert runner._graphs, "no step was replayed from a graph"
    for r in rids:
        runner.finish(r)
    runner.cache.check_invariants()
