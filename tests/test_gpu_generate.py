"""Generation through the entry point: ``LLM.generate`` drives scheduler, step function, cache
and sampling kernels; the plain implementation re-runs the whole sequence for every token."""

import pytest
import torch

import parity
from plain_model import plain_forward, plain_load
from plain_sampler import plain_sample
from rapid_llm_amd.sampling.rng import uniform_draw
from tiny_configs import TINY, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu


def _llm(model_dir, dtype, page, **kw):
    from rapid_llm_amd import LLM

    body = dict(dtype=dtype, page_size=page, num_pages=200, max_num_seqs=8, use_cuda_graph=False)
    body.update(kw)
    return LLM(str(model_dir), **body)


def _plain_generate(cfg, w, prompt, n, temperature=0.0, top_p=1.0, seed=0, penalty=1.0):
    ids, out = list(prompt), []
    for i in range(n):
        logits = plain_forward(cfg, w, ids)[-1]
        tok = plain_sample(logits, temperature, top_p, uniform_draw(seed, i), penalty, out)
        out.append(tok)
        ids.append(tok)
    return out


def test_greedy_generation_tiny_a_float32(tmp_path):
    """Tiny configuration A: prompts of 1/5/13/29 tokens, 12 greedy tokens each."""
    from rapid_llm_amd import SamplingParams

    cfg, page, seed = TINY["A"]
    model_dir = make_model_dir(tmp_path, "A", "float32")
    pcfg, pw = plain_load(model_dir)
    prompts = [random_tokens(n, cfg["vocab_size"], seed + n) for n in (1, 5, 13, 29)]
    llm = _llm(model_dir, "float32", page, max_seq_len=128)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_gen_len=12))
    for prompt, out in zip(prompts, outs):
        assert out.outputs[0].token_ids == _plain_generate(pcfg, pw, prompt, 12)
        assert out.outputs[0].finish_reason == "length" and out.prompt_token_ids == prompt
    # batched == one by one, and run-to-run equal (tests/engine/test_engine_e2e.py:27-83)
    for prompt, out in zip(prompts, outs):
        alone = llm.generate(prompt, SamplingParams(temperature=0.0, max_gen_len=12))
        assert alone[0].token_ids == out.token_ids
    llm.scheduler.cache.check_invariants()
    assert not llm.scheduler.cache.live_requests()


def test_sampled_generation_tiny_b_chunked_and_mixed(tmp_path):
    """Tiny configuration B: prompts of 2/17/31/64/90/150 tokens in portions of 24 mixed
    with decodes, then 20 tokens each at temperature 0.8 with a fixed seed."""
    from rapid_llm_amd import SamplingParams

    cfg, page, seed = TINY["B"]
    model_dir = make_model_dir(tmp_path, "B", "float32")
    pcfg, pw = plain_load(model_dir)
    prompts = [random_tokens(n, cfg["vocab_size"], seed + n) for n in (2, 17, 31, 64, 90, 150)]
    llm = _llm(model_dir, "float32", page, max_seq_len=256, max_chunk_size=24, max_num_batched_tokens=64,
               max_num_seqs=4)
    params = [SamplingParams(temperature=0.8, top_p=0.9, max_gen_len=20, seed=77 + i, logprobs=0)
              for i in range(len(prompts))]
    outs = llm.generate(prompts, params)
    mixed_steps = 0
    for i, (prompt, out) in enumerate(zip(prompts, outs)):
        want = _plain_generate(pcfg, pw, prompt, 20, 0.8, 0.9, 77 + i)
        assert out.token_ids == want, i
        records = out.outputs[0].logprobs
        assert [r.token_id for r in records] == want and all(r.logprob <= 0 and not r.top_token_ids for r in records)
    # the same requests, unchunked and one at a time, draw the same tokens
    solo = _llm(model_dir, "float32", page, max_seq_len=256, max_chunk_size=0, max_num_batched_tokens=256,
                max_num_seqs=1)
    for prompt, p, out in zip(prompts, params, outs):
        assert solo.generate(prompt, p)[0].token_ids == out.token_ids


@pytest.mark.parametrize("which,pages", [("A", 24), ("C", 13)])
def test_eviction_changes_nothing(tmp_path, which, pages):
    """So few pages that running requests are evicted and recomputed: the tokens are the ones
    an ample pool gives, greedy and sampled.  Configuration C has windowed layers beside a
    full one: two pools, of which the windowed one gives pages back while requests run."""
    from rapid_llm_amd import SamplingParams

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, "float32")
    prompts = [random_tokens(n, cfg["vocab_size"], seed + n) for n in (9, 14, 6, 11)]
    params = [SamplingParams(temperature=0.0 if i % 2 else 0.7, top_p=0.95, max_gen_len=30, seed=i,
                             repetition_penalty=1.15) for i in range(4)]
    ample = _llm(model_dir, "float32", page, max_seq_len=128).generate(prompts, params)
    tight = _llm(model_dir, "float32", page, max_seq_len=128, num_pages=pages)  # room for about two requests
    outs = tight.generate(prompts, params)
    assert tight.scheduler.num_preemptions > 0
    assert [o.token_ids for o in outs] == [o.token_ids for o in ample]
    cache = tight.scheduler.cache
    cache.check_invariants()
    assert all(pool.num_free == pages - 1 for pool in cache.pools.values())
    assert len(cache.pools) == (2 if which == "C" else 1)


def test_logprob_records_of_prompt_and_output(tmp_path):
    """Prompt positions are scored on the raw logits, generated tokens on the distribution
    they were drawn from; portions of 5 tokens beside decoded tokens, and a pool so small
    that requests are evicted and run again, change no record."""
    from plain_sampler import plain_logprob, plain_top_logprobs
    from rapid_llm_amd import SamplingParams

    cfg, page, seed = TINY["A"]
    model_dir = make_model_dir(tmp_path, "A", "float32")
    pcfg, pw = plain_load(model_dir)
    prompts = [random_tokens(n, cfg["vocab_size"], seed + 3 * n) for n in (1, 12, 7)]
    params = [
        SamplingParams(temperature=0.0, max_gen_len=9, logprobs=3, prompt_logprobs=2),
        SamplingParams(temperature=0.9, top_p=0.9, max_gen_len=9, seed=5, logprobs=2, prompt_logprobs=4,
                       repetition_penalty=1.2),
        SamplingParams(temperature=0.7, top_p=1.0, max_gen_len=9, seed=6, logprobs=0),
    ]
    llm = _llm(model_dir, "float32", page, max_seq_len=128, max_chunk_size=5, max_num_batched_tokens=12)
    outs = llm.generate(prompts, params)
    tight = _llm(model_dir, "float32", page, max_seq_len=128, max_chunk_size=5, max_num_batched_tokens=12,
                 num_pages=9)
    evicted = tight.generate(prompts, params)
    assert tight.scheduler.num_preemptions > 0

    def near(a, b):
        return abs(a - b) < 1e-4 * max(1.0, abs(b))

    for prompt, p, out, again in zip(prompts, params, outs, evicted):
        tokens = out.token_ids
        assert again.token_ids == tokens
        logits = plain_forward(pcfg, pw, prompt + tokens)
        if p.prompt_logprobs is None:
            assert out.prompt_logprobs is None
        else:
            assert len(out.prompt_logprobs) == len(prompt) and out.prompt_logprobs[0] is None
            for q in range(1, len(prompt)):
                rec = out.prompt_logprobs[q]
                assert rec.token_id == prompt[q]
                assert near(rec.logprob, plain_logprob(logits[q - 1], prompt[q], 1.0))
                ids, lps = plain_top_logprobs(logits[q - 1], p.prompt_logprobs)
                assert list(rec.top_token_ids) == ids and all(near(a, b) for a, b in zip(rec.top_logprobs, lps))
        records = out.outputs[0].logprobs
        assert [r.token_id for r in records] == tokens
        for i, rec in enumerate(records):
            row = logits[len(prompt) - 1 + i]
            args = (p.temperature, p.repetition_penalty, tokens[:i])
            assert near(rec.logprob, plain_logprob(row, tokens[i], *args))
            ids, lps = plain_top_logprobs(row, p.logprobs, *args)
            assert list(rec.top_token_ids) == ids and all(near(a, b) for a, b in zip(rec.top_logprobs, lps))
        for mine, theirs in zip(records, again.outputs[0].logprobs):
            assert mine.token_id == theirs.token_id and near(mine.logprob, theirs.logprob)
        if p.prompt_logprobs is not None:
            assert [r and r.token_id for r in again.prompt_logprobs] == [r and r.token_id for r in out.prompt_logprobs]


@pytest.mark.parametrize("which", ["A", "B", "C", "D", "F", "H"])
def test_bfloat16_generation_stays_near_the_plain_choice(tmp_path, which):
    from rapid_llm_amd import SamplingParams

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, "bfloat16")
    pcfg, pw = plain_load(model_dir)
    prompts = [random_tokens(n, cfg["vocab_size"], seed + n) for n in (3, 20, 45)]
    for graph in (False, True):
        llm = _llm(model_dir, "bfloat16", page, max_seq_len=cfg["max_position_embeddings"], use_cuda_graph=graph)
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_gen_len=16))
        for prompt, out in zip(prompts, outs):
            ids = list(prompt)
            for tok in out.token_ids:
                parity.assert_near_choice(plain_forward(pcfg, pw, ids)[-1], tok, f"{which}/graph={graph}")
                ids.append(tok)
            assert len(out.token_ids) == 16


@pytest.mark.parametrize("which,count,rows", [("E", 40, (17, 64)), ("D", 100, (65, 128))])
def test_bfloat16_generation_of_many_requests_at_once(tmp_path, which, count, rows):
    """Decode batches between 17 and 64 rows (configuration E: the output and down projections
    then run as runs of K added by the norms) and beyond 64 (every product from the library),
    with and without graphs."""
    from rapid_llm_amd import SamplingParams

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, "bfloat16")
    pcfg, pw = plain_load(model_dir)
    prompts = [random_tokens(2 + (7 * i) % 23, cfg["vocab_size"], seed + i) for i in range(count)]
    for graph in (False, True):
        llm = _llm(model_dir, "bfloat16", page, max_seq_len=64, max_num_seqs=count + 8,
                   num_pages=(count + 8) * (64 // page) + 8, use_cuda_graph=graph)
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_gen_len=6))
        for prompt, out in zip(prompts, outs):
            ids = list(prompt)
            for tok in out.token_ids:
                parity.assert_near_choice(plain_forward(pcfg, pw, ids)[-1], tok, f"{which}/{count}/graph={graph}")
                ids.append(tok)
            assert len(out.token_ids) == 6
        if graph:
            assert any(rows[0] <= key[0] <= rows[1] for key in llm.scheduler.runner._graphs)


def test_stop_tokens_and_stream(tmp_path):
    from rapid_llm_amd import LLM, SamplingParams

    cfg, page, seed = TINY["A"]
    model_dir = make_model_dir(tmp_path, "A", "float32")
    prompt = random_tokens(7, cfg["vocab_size"], 5)
    free = _llm(model_dir, "float32", page, max_seq_len=64).generate(prompt, SamplingParams(temperature=0.0, max_gen_len=10))[0]
    stop = free.token_ids[4]
    (model_dir / "generation_config.json").write_text('{"eos_token_id": [%d]}' % stop)
    llm = _llm(model_dir, "float32", page, max_seq_len=64)
    out = llm.generate(prompt, SamplingParams(temperature=0.0, max_gen_len=10))[0]
    first = free.token_ids.index(stop)
    assert out.token_ids == free.token_ids[:first] and out.outputs[0].finish_reason == "eos"
    seen = []
    for batch in llm.stream([prompt, prompt[:3]], SamplingParams(temperature=0.0, max_gen_len=5, ignore_eos=True)):
        seen.append([len(o.token_ids) for o in batch])
    assert seen[-1] == [5, 5] or seen[-1] == [5]
    assert sum(1 for s in seen) >= 5


@pytest.mark.parametrize("dtype,graph", [("float32", False), ("bfloat16", True)])
def test_pipeline_gives_the_tokens_of_the_synchronous_loop(tmp_path, dtype, graph):
    """Steps queued before the last one's tokens are read (decoded tokens fed from the device,
    stop tokens seen a step late) against every step read before the next is planned: greedy
    and sampled requests, a stop token, portions beside decoded tokens, few pages."""
    from rapid_llm_amd import SamplingParams

    cfg, page, seed = TINY["B"]
    model_dir = make_model_dir(tmp_path, "B", dtype)
    prompts = [random_tokens(n, cfg["vocab_size"], seed + 7 * n) for n in (3, 40, 1, 19, 26, 8)]
    params = [SamplingParams(temperature=0.0 if i % 2 == 0 else 0.8, top_p=0.9, max_gen_len=6 + 5 * i, seed=i,
                             logprobs=1 if i == 1 else None)
              for i in range(len(prompts))]
    common = dict(max_seq_len=128, max_chunk_size=16, max_num_batched_tokens=40, max_num_seqs=4,
                  use_cuda_graph=graph)
    free = _llm(model_dir, dtype, page, pipeline=False, **common).generate(prompts, params)
    stop = free[4].token_ids[9]
    (model_dir / "generation_config.json").write_text('{"eos_token_id": [%d]}' % stop)
    outs = {}
    for pipeline in (False, True):
        for pages in (200, 8):
            llm = _llm(model_dir, dtype, page, pipeline=pipeline, num_pages=pages, **common)
            assert llm.scheduler.pipeline == pipeline
            outs[pipeline, pages] = llm.generate(prompts, params)
            llm.scheduler.cache.check_invariants()
            assert not llm.scheduler.cache.live_requests() and not llm.scheduler._held
            if pages == 8:
                assert llm.scheduler.num_preemptions > 0
    base = outs[False, 200]
    assert dtype == "bfloat16" or any(o.outputs[0].finish_reason == "eos" for o in base)
    pcfg, pw = plain_load(model_dir)
    for key, got in outs.items():
        if dtype == "bfloat16":
            # another schedule puts a token into a step of another shape, which other kernels
            # run: it rounds differently, so a near-tie may fall the other way and a sampled
            # request may draw another token.  float32 is exact; here every greedy request's
            # tokens must lie within rounding of the plain choice given its own tokens so far,
            # a request ends by a stop token exactly when it produced one, and the others by count.
            for i, (prompt, p, o) in enumerate(zip(prompts, params, got)):
                reason = o.outputs[0].finish_reason
                assert reason in ("length", "eos") and (o.token_ids or reason == "eos"), key
                assert stop not in o.token_ids, key
                assert reason == "eos" or len(o.token_ids) == p.max_gen_len, key
                if p.temperature == 0.0:
                    ids = list(prompt)
                    for tok in o.token_ids:
                        parity.assert_near_choice(plain_forward(pcfg, pw, ids)[-1], tok, f"pipeline {key} request {i}")
                        ids.append(tok)
                    if reason == "eos":  # what ended it was a choice within rounding of the plain one too
                        parity.assert_near_choice(plain_forward(pcfg, pw, ids)[-1], stop, f"pipeline {key} request {i} stop")
            continue
        for a, b in zip(base, got):
            assert a.token_ids == b.token_ids and a.outputs[0].finish_reason == b.outputs[0].finish_reason, key
            if a.outputs[0].logprobs is not None:
                assert [r.token_id for r in a.outputs[0].logprobs] == [r.token_id for r in b.outputs[0].logprobs]


def test_a_repetition_penalty_rides_the_pipeline(tmp_path):
    """With a penalty the newest token of a request is part of what the next choice depends
    on; pipelined, that token is still on the device.  Tokens and records are those of the
    synchronous loop and of the plain model and sampler, with ample pages and with few."""
    from rapid_llm_amd import SamplingParams

    cfg, page, seed = TINY["A"]
    model_dir = make_model_dir(tmp_path, "A", "float32")
    cfg, w = plain_load(model_dir)
    prompts = [random_tokens(n, cfg["vocab_size"], seed + 3 * n) for n in (5, 21, 2, 13, 30)]
    params = [SamplingParams(temperature=0.0 if i % 2 == 0 else 0.9, top_p=0.95, max_gen_len=10 + 3 * i, seed=i,
                             repetition_penalty=1.0 if i == 3 else 6.0 + 0.5 * i, stop_on_repeat=False,
                             logprobs=2 if i == 0 else None)
              for i in range(len(prompts))]
    common = dict(max_seq_len=128, max_chunk_size=16, max_num_batched_tokens=40, max_num_seqs=4,
                  use_cuda_graph=False)
    outs = {}
    for pipeline in (False, True):
        for pages in (200, 18):  # 17 pages of 4: the longest request alone fits, four together do not
            llm = _llm(model_dir, "float32", page, pipeline=pipeline, num_pages=pages, **common)
            outs[pipeline, pages] = llm.generate(prompts, params)
            assert not llm.scheduler.cache.live_requests() and not llm.scheduler._held
            if pages == 18:
                assert llm.scheduler.num_preemptions > 0
    base = outs[False, 200]
    for prompt, p, o in zip(prompts, params, base):
        if p.temperature == 0.0:  # a sampled row may sit within rounding of another token
            want = _plain_generate(cfg, w, prompt, p.max_gen_len, penalty=p.repetition_penalty)
            assert o.token_ids == want
            if p.repetition_penalty > 1.0:
                assert len(set(want)) > len(want) // 2, "the penalty changed nothing to see"
    greedy_free = _plain_generate(cfg, w, prompts[0], params[0].max_gen_len)
    assert greedy_free != base[0].token_ids, "the penalty made no difference to the tokens"
    for key, got in outs.items():
        for a, b in zip(base, got):
            assert a.token_ids == b.token_ids, key
            if a.outputs[0].logprobs is not None:
                assert [(r.token_id, r.top_token_ids) for r in a.outputs[0].logprobs] == \
                       [(r.token_id, r.top_token_ids) for r in b.outputs[0].logprobs], key


def test_command_line_batch(tmp_path, capsys):
    from rapid_llm_amd.cli import main

    cfg, page, seed = TINY["B"]
    model_dir = make_model_dir(tmp_path, "B", "float32")
    prompts = tmp_path / "prompts.txt"
    prompts.write_text("[1, 2, 3, 4]\n\n[10, 20]\n")
    code = main(["batch", "--model-dir", str(model_dir), "--dtype", "float32", "--max-seq-len", "64",
                 "--temperature", "0", "--max-gen-len", "6", "--repetition-penalty", "1.0",
                 "--prompts-file", str(prompts), "--show-stats", "--no-cuda-graph"])
    text = capsys.readouterr().out
    assert code == 0 and "--- [0] length ---" in text and "--- [1] length ---" in text
    assert "2 requests, 12 tokens" in text and "throughput" in text
    pcfg, pw = plain_load(model_dir)
    assert str(_plain_generate(pcfg, pw, [1, 2, 3, 4], 6)) in text


def test_entry_point_options(tmp_path):
    """What ``LLM(...)`` takes beside the model folder: options of the reference that this
    engine has no use for are refused by name; the cache pool comes from the reference's knob
    (in tokens), or from the memory that is free, capped at what every slot at full length can
    use; ``hf_overrides`` changes configuration keys; ``load_format="random"`` needs no
    weights file and is fixed by the seed."""
    from rapid_llm_amd import LLM, SamplingParams

    cfg, page, seed = TINY["B"]
    model_dir = make_model_dir(tmp_path, "B", "float32")
    for kw, message in ((dict(quantization="int8"), "quantization"), (dict(tensor_parallel_size=2), "one GPU"),
                        (dict(data_parallel_size=4), "one GPU"), (dict(kv_cache_dtype="fp8"), "kv_cache_dtype")):
        with pytest.raises(ValueError, match=message):
            LLM(str(model_dir), **kw)
    common = dict(dtype="float32", max_seq_len=64, page_size=8, max_num_seqs=4, use_cuda_graph=False)
    assert LLM(str(model_dir), max_gpu_num_blocks=200, **common).scheduler.cache.pools[0].num_usable == 25
    assert LLM(str(model_dir), **common).scheduler.cache.pools[0].num_usable == 4 * 8
    # two of the three layers: the plain model with the same key changed
    prompt = random_tokens(9, cfg["vocab_size"], 3)
    params = SamplingParams(temperature=0.0, max_gen_len=8)
    pcfg, pw = plain_load(model_dir)
    short = LLM(str(model_dir), hf_overrides={"num_hidden_layers": 2}, **common).generate(prompt, params)[0]
    assert short.token_ids == _plain_generate(dict(pcfg, num_hidden_layers=2), pw, prompt, 8)
    assert short.token_ids != _plain_generate(pcfg, pw, prompt, 8)
    # random weights from a configuration alone
    outs = [LLM(dict(cfg), load_format="random", seed=s, **common).generate(prompt, params)[0].token_ids
            for s in (3, 3, 4)]
    assert outs[0] == outs[1] and outs[0] != outs[2]


def _word_tokenizer(model_dir, vocab):
    """A tokenizer.json in which the word ``w<i>`` is token ``i``."""
    from tokenizers import Tokenizer, models, pre_tokenizers

    tok = Tokenizer(models.WordLevel({f"w{i}": i for i in range(vocab)}, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.save(str(model_dir / "tokenizer.json"))


def test_text_prompts_with_a_tokenizer(tmp_path, capsys, monkeypatch):
    """A model folder with a tokenizer.json takes text and gives text back: through
    ``generate``, through ``stream`` (whose deltas add up to the text), and through the
    ``batch`` and ``chat`` commands."""
    from rapid_llm_amd import SamplingParams
    from rapid_llm_amd.cli import main

    cfg, page, seed = TINY["A"]
    model_dir = make_model_dir(tmp_path, "A", "float32")
    _word_tokenizer(model_dir, cfg["vocab_size"])
    llm = _llm(model_dir, "float32", page, max_seq_len=64)
    params = SamplingParams(temperature=0.0, max_gen_len=6)
    by_text = llm.generate(["w5 w17 w3", "w9"], params)
    by_ids = llm.generate([[5, 17, 3], [9]], params)
    for a, b in zip(by_text, by_ids):
        assert a.prompt_token_ids == b.prompt_token_ids and a.token_ids == b.token_ids
        assert a.text == " ".join(f"w{t}" for t in a.token_ids)
    assert by_text[0].prompt == "w5 w17 w3"
    texts = [batch[0].text for batch in llm.stream("w5 w17 w3", params)]
    assert texts[-1] == by_text[0].text and len(texts) >= 6
    assert all(later.startswith(earlier) for earlier, later in zip(texts, texts[1:]))
    prompts = tmp_path / "prompts.txt"
    prompts.write_text("w5 w17 w3\nw9\n")
    common = ["--model-dir", str(model_dir), "--dtype", "float32", "--max-seq-len", "64", "--temperature", "0",
              "--max-gen-len", "6", "--repetition-penalty", "1.0", "--no-cuda-graph"]
    assert main(["batch", *common, "--prompts-file", str(prompts), "--no-chat-template"]) == 0
    text = capsys.readouterr().out
    assert by_text[0].text in text and by_text[1].text in text
    lines = iter(["w5 w17 w3", "/clear", "", "w9", "exit"])
    monkeypatch.setattr("builtins.input", lambda prompt="": next(lines))
    assert main(["chat", *common]) == 0
    text = capsys.readouterr().out
    assert text.count("w") > 10  # two streamed answers of six words each


def test_the_page_pool_is_what_memory_is_left_and_a_budget_of_nothing_is_refused(tmp_path):
    """Without ``num_pages`` the pool is sized from the free memory less the state tensors and
    the recorded steps' estimate; a utilisation that leaves nothing raises instead of making a
    pool of two pages."""
    from rapid_llm_amd import EngineConfig, ModelRunner

    cfg, page, seed = TINY["B"]
    model_dir = make_model_dir(tmp_path, "B", "bfloat16")
    free, total = torch.cuda.mem_get_info()
    common = dict(dtype="bfloat16", max_seq_len=128, page_size=page, max_num_seqs=4)
    runner = ModelRunner(model_dir, EngineConfig(**common))
    assert runner.cache.pools[0].num_usable == 4 * (128 // page)  # capped: every slot at full length
    estimate = runner._graph_pool_estimate()
    assert estimate > 0 and runner.state_bytes == 0
    assert ModelRunner(model_dir, EngineConfig(use_graph=False, **common))._graph_pool_estimate() == 0
    # a batch is padded up to the next size of the ladder: five requests record eight rows, and
    # the split results that the decode attention keeps between its kernels are counted
    by_seqs = {
        n: ModelRunner(model_dir, EngineConfig(**dict(common, max_num_seqs=n, num_pages=8)))._graph_pool_estimate()
        for n in (4, 5, 8)
    }
    assert by_seqs[5] == by_seqs[8] > by_seqs[4]
    mixer = runner.model.blocks[0].mixer
    assert mixer.recorded_step_bytes(1, 128, page) == 0  # too few keys to split
    kept = mixer.recorded_step_bytes(1, 4096, page)
    assert kept == 1 * cfg["num_attention_heads"] * 32 * (cfg["head_dim"] + 2) * 4  # 32 splits of 128 keys
    # keep back more than is free: nothing is left for pages
    too_little = max(1e-6, min(0.5, 0.5 * free / total) * 1e-3)
    with pytest.raises(ValueError, match="no memory is left for the cache"):
        ModelRunner(model_dir, EngineConfig(gpu_memory_utilization=too_little, **common))
    # a pool of a given size that cannot be made says so, and how many pages can, before anything
    # is allocated
    per_page = sum(runner.page_bytes.values())
    with pytest.raises(ValueError, match=r"a cache of \d+ pages .* ask for at most \d+ pages"):
        ModelRunner(model_dir, EngineConfig(num_pages=total // per_page + 2, **common))
    with pytest.raises(ValueError, match="ask for at most"):
        ModelRunner(model_dir, EngineConfig(max_gpu_num_blocks=(total // per_page + 2) * page, **common))


def test_template_and_stop_token_of_the_model_folder(tmp_path, capsys):
    """``batch`` formats prompts with the folder's chat template, and a token that only
    ``tokenizer_config.json`` names as the end of a sequence ends one."""
    import json

    from rapid_llm_amd import SamplingParams
    from rapid_llm_amd.cli import main

    cfg, page, seed = TINY["A"]
    model_dir = make_model_dir(tmp_path, "A", "float32")
    _word_tokenizer(model_dir, cfg["vocab_size"])
    params = SamplingParams(temperature=0.0, max_gen_len=6)
    free = _llm(model_dir, "float32", page, max_seq_len=64).generate(["w7 w5 w17 w3 w8"], params)[0]
    assert free.outputs[0].finish_reason == "length"
    stop = free.token_ids[-1]
    first = free.token_ids.index(stop)
    (model_dir / "tokenizer_config.json").write_text(json.dumps({
        "eos_token": f"w{stop}",
        "chat_template": "w7 {{ messages[0]['content'] }}{% if add_generation_prompt %} w8{% endif %}",
    }))
    stopped = _llm(model_dir, "float32", page, max_seq_len=64).generate(["w7 w5 w17 w3 w8"], params)[0]
    assert stopped.outputs[0].finish_reason == "eos" and stopped.token_ids == free.token_ids[:first]
    prompts = tmp_path / "prompts.txt"
    prompts.write_text("w5 w17 w3\n")
    common = ["--model-dir", str(model_dir), "--dtype", "float32", "--max-seq-len", "64", "--temperature", "0",
              "--max-gen-len", "6", "--repetition-penalty", "1.0", "--no-cuda-graph", "--prompts-file", str(prompts)]
    assert main(["batch", *common]) == 0
    text = capsys.readouterr().out
    assert "[0] eos" in text and stopped.text in text  # the template wrapped the line as the text prompt above
    assert main(["batch", *common, "--no-chat-template"]) == 0


def test_command_line_defaults_and_replay(tmp_path, capsys, monkeypatch):
    """``batch`` with the command line's own defaults (temperature 0.6, nucleus 0.9, penalty
    1.1, graphs, the folder from the environment) ends every request; ``replay`` writes the
    logits ``bin/trace_run`` would."""
    import json

    import numpy as np

    from rapid_llm_amd.cli import main

    cfg, page, seed = TINY["D"]
    model_dir = make_model_dir(tmp_path, "D", "bfloat16")
    monkeypatch.setenv("RAPID_LLM_MODEL_DIR", str(model_dir))
    assert main(["batch", "--max-seq-len", "96", "--max-gen-len", "40", "--show-stats"]) == 0
    text = capsys.readouterr().out
    assert text.count("--- [") == 4 and "4 requests" in text
    trace = tmp_path / "trace.jsonl"
    toks = random_tokens(20, cfg["vocab_size"], 1)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:17], "want": [16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[17:], "want": [0, 2]}], "end": ["a"]}]
    trace.write_text("".join(json.dumps(s) + "\n" for s in steps))
    out = tmp_path / "logits"
    assert main(["replay", "--model", str(model_dir), "--dtype", "float32", "--out", str(out), "--max-tokens", "64",
                 "--trace", str(trace)]) == 0
    assert capsys.readouterr().out.split() == ["done", "0", "done", "1"]
    pcfg, pw = plain_load(model_dir)
    want = plain_forward(pcfg, pw, toks)
    got = np.fromfile(out / "1.f32", dtype="<f4").reshape(2, cfg["vocab_size"])
    assert np.allclose(got, want[[17, 19]].numpy(), rtol=2e-5, atol=3e-6)


def test_command_line_bench(tmp_path, capsys):
    import json

    from rapid_llm_amd.cli import main

    model_dir = make_model_dir(tmp_path, "D", "bfloat16")
    code = main(["bench", "--model-dir", str(model_dir), "--max-seq-len", "128", "--batch-size", "5",
                 "--input-len", "40", "--gen-len", "12", "--iterations", "2", "--warmup", "1"])
    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert code == 0 and line["batch_size"] == 5 and line["tgs"] > 0 and line["ttft_s"] > 0 and line["tpot_ms"] > 0
    assert line["input_len_min"] == line["input_len_max"] == 40
    # prompt lengths drawn from a range, as the reference's random dataset draws them
    code = main(["bench", "--model-dir", str(model_dir), "--max-seq-len", "128", "--batch-size", "6",
                 "--input-len-min", "3", "--input-len-max", "70", "--gen-len", "9", "--iterations", "1", "--warmup", "0"])
    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert code == 0 and (line["input_len_min"], line["input_len_max"]) == (3, 70) and line["tgs"] > 0
    code = main(["bench", "--model-dir", str(model_dir), "--max-seq-len", "128", "--batch-size", "3",
                 "--input-len", "64", "--range-ratio", "0.25", "--gen-len", "5", "--iterations", "1", "--warmup", "0"])
    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert code == 0 and (line["input_len_min"], line["input_len_max"]) == (16, 64)


def test_command_line_bench_profile(tmp_path, capsys):
    """``--profile`` prints the device time of every part by kind of step: every part of the
    model is there, the decode steps were timed eagerly, and the regions add up to their total."""
    import json
    import re

    from rapid_llm_amd.cli import main

    model_dir = make_model_dir(tmp_path, "D", "bfloat16")
    code = main(["bench", "--model-dir", str(model_dir), "--max-seq-len", "128", "--batch-size", "3",
                 "--input-len", "20", "--gen-len", "6", "--iterations", "1", "--warmup", "0", "--profile"])
    shown = capsys.readouterr()
    assert code == 0 and json.loads(shown.out.strip().splitlines()[-1])["tgs"] > 0
    table = shown.err
    assert "steps with prompt portions:" in table and "decode steps:" in table
    decode = table.split("decode steps:")[1]
    for region in ("embedding (TokenEmbedding)", "mixer norm (RMSNorm)", "mixer (GQAAttention)",
                   "feed-forward norm (RMSNorm)", "feed-forward (SwiGLU)", "final norm (RMSNorm)",
                   "output projection (LinearOutput)"):
        assert region in decode, f"{region} is missing:\n{table}"
    # five decode steps of a two-layer model: ten calls of every part of a layer, five of the ends
    calls = {m.group(1).strip(): int(m.group(2)) for m in re.finditer(r"^  (.+?)\s+(\d+) calls", decode, re.M)}
    assert calls["mixer (GQAAttention)"] == 10 and calls["output projection (LinearOutput)"] == 5
    total = float(re.search(r"^\s*([0-9.]+) ms inside parts", decode, re.M).group(1))
    parts = sum(float(m.group(1)) for m in re.finditer(r"calls\s+([0-9.]+) ms", decode))
    assert abs(parts - total) < 0.01 * total + 0.01


def test_smoke_entry():
    import __graft_entry__

    __graft_entry__.smoke()
