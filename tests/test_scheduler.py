"""The scheduler's decisions, with a scripted step function in place of the model (CPU only).

The pattern is the reference's ``_ScriptedExecutor`` (tests/engine/test_scheduler.py:46-74,
tests/engine/test_batch_planner.py:156-610)."""

import dataclasses

import pytest

from rapid_llm_amd.cache import CacheManager, GroupSpec
from rapid_llm_amd.config import EngineConfig
from rapid_llm_amd.engine.feed import fed_row, fed_token
from rapid_llm_amd.engine.request import RequestStatus
from rapid_llm_amd.engine.scheduler import Scheduler, StepOutput, detect_repetition
from rapid_llm_amd.sampling import PositionLogprobs, SamplingParams

EOS = 99


class ScriptedExecutor:
    """Checks that every step is runnable from what the plan reserved, records its shape,
    and "samples" token ``f(request, index of the output token)``; a row with a repetition
    penalty takes the next id that its history does not hold, so its tokens depend on all
    the tokens before."""

    def __init__(self, num_pages, page, seqs, max_len, window=0, token=None):
        self.cache = CacheManager([GroupSpec(0, window, (0,))], num_pages, page, seqs, max_len)
        self.token = token or (lambda rid, i: 1000 + i)
        self.steps = []
        self.wants = []  # (request, first position, tokens, wanted places) of every entry run
        self.computed = {}
        self.fed = {}

    def execute(self, entries, sampling):
        rows = sampling.rows
        shape, out = [], []
        k = 0
        num_rows = 0
        for e in entries:
            assert self.cache.has(e.request_id), "an entry without a slot"
            start = self.computed.get(e.request_id, 0)
            assert self.cache.reserved(e.request_id) >= start + len(e.tokens), "pages were not reserved"
            self.computed[e.request_id] = start + len(e.tokens)
            self.fed.setdefault(e.request_id, []).extend(e.tokens)
            shape.append((e.request_id, len(e.tokens), bool(e.want)))
            self.wants.append((e.request_id, start, len(e.tokens), list(e.want)))
            if e.want and k < len(rows) and sampling.logits_rows[k] == num_rows + len(e.want) - 1:
                assert e.want[-1] == len(e.tokens) - 1
                token = self.token(e.request_id, rows[k].counter)
                if rows[k].repetition_penalty != 1.0:
                    assert len(rows[k].generated) == rows[k].counter, "the history misses a token"
                    assert min(rows[k].generated, default=0) >= 0, "a history token nobody resolved"
                    while token != EOS and token in rows[k].generated:
                        token = (token + 1) % 50
                out.append(token)
                k += 1
            num_rows += len(e.want)
        assert k == len(rows)
        self.steps.append(shape)
        self.cache.check_invariants()
        result = StepOutput(out)
        if any(kk is not None for kk in sampling.logprob_ks):
            result.logprobs = [
                None if kk is None else PositionLogprobs(t, -1.0, tuple(range(kk)), (-2.0,) * kk)
                for t, kk in zip(out, sampling.logprob_ks)
            ]
        if sampling.prompt_rows:
            assert max(sampling.prompt_rows) < num_rows
            result.prompt_logprobs = [
                PositionLogprobs(t, -float(row), tuple(range(kk)), (-2.0,) * kk)
                for row, t, kk in zip(sampling.prompt_rows, sampling.prompt_targets, sampling.prompt_ks)
            ]
        return result

    def finish(self, request_id):
        self.cache.release(request_id)
        self.computed.pop(request_id, None)
        self.fed.pop(request_id, None)


class PipelinedExecutor(ScriptedExecutor):
    """The same, with ``launch``: the result of a step may be read after the next step has
    been queued.  A fed token must name the row of the previous launch in which its own
    request was sampled; it is replaced by what that row chose, as the device would."""

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.previous = []  # (request id, token) per sampling row of the latest launch
        self.unread = 0
        self.max_unread = 0
        self.history = {}  # every token fed for a request, over its evictions too: position -> token

    def launch(self, entries, sampling):
        resolved = []
        for e in entries:
            tokens = list(e.tokens)
            if tokens[0] < 0:
                assert len(tokens) == 1, "only a single token can be fed from the device"
                rid, token = self.previous[fed_row(tokens[0])]
                assert rid == e.request_id, "a fed token names another request's row"
                tokens = [token]
            assert min(tokens) >= 0
            start = self.computed.get(e.request_id, 0)
            for i, t in enumerate(tokens):
                assert self.history.setdefault((e.request_id, start + i), t) == t, "a position changed its token"
            resolved.append(type(e)(e.request_id, tokens, e.want))
        # a penalised row's history may name its newest token the same way
        sampled_rids = []
        num_rows, k = 0, 0
        for e in entries:
            if k < len(sampling.rows) and e.want and sampling.logits_rows[k] == num_rows + len(e.want) - 1:
                sampled_rids.append(e.request_id)
                k += 1
            num_rows += len(e.want)
        rows = []
        for rid, row in zip(sampled_rids, sampling.rows):
            history = list(row.generated)
            assert all(t >= 0 for t in history[:-1]), "only the newest token can be pending"
            if history and history[-1] < 0:
                owner, token = self.previous[fed_row(history[-1])]
                assert owner == rid, "a history names another request's row"
                history[-1] = token
            rows.append(dataclasses.replace(row, generated=history))
        sampling = dataclasses.replace(sampling, rows=rows)
        result = self.execute(resolved, sampling)
        self.previous = list(zip(sampled_rids, result.token_ids))
        self.unread += 1
        self.max_unread = max(self.max_unread, self.unread)
        executor = self

        class Handle:
            def result(self_inner):
                executor.unread -= 1
                return result

        return Handle()


def _make_pipelined(num_pages=64, page=4, seqs=4, max_len=128, token=None, pipeline=True, **cfg):
    ex = PipelinedExecutor(num_pages, page, seqs, max_len, token=token)
    config = EngineConfig(max_seq_len=max_len, page_size=page, num_pages=num_pages, max_num_seqs=seqs,
                          pipeline=pipeline, **{"max_num_batched_tokens": 64, "max_chunk_size": 16, **cfg})
    return Scheduler(ex, config, stop_token_ids=[EOS]), ex


def _make(num_pages=64, page=4, seqs=4, max_len=128, token=None, **cfg):
    ex = ScriptedExecutor(num_pages, page, seqs, max_len, token=token)
    config = EngineConfig(max_seq_len=max_len, page_size=page, num_pages=num_pages, max_num_seqs=seqs,
                          **{"max_num_batched_tokens": 64, "max_chunk_size": 16, **cfg})
    return Scheduler(ex, config, stop_token_ids=[EOS]), ex


GREEDY = SamplingParams(temperature=0.0, max_gen_len=4)


def test_submission_rules():
    s, _ = _make(max_len=32)
    with pytest.raises(ValueError, match="empty"):
        s.add_request([], GREEDY)
    with pytest.raises(ValueError, match="no room"):
        s.add_request(list(range(32)), GREEDY)
    with pytest.raises(ValueError, match="tokenizer"):
        s.add_request("text", GREEDY)
    r = s.add_request(list(range(30)), SamplingParams(temperature=0.0, max_gen_len=10))
    assert r.max_new_tokens == 2  # capped by the context (batch_planner.py:403-427)
    assert s.add_request([1], SamplingParams(temperature=0.0)).max_new_tokens == 31
    s.add_request([1], GREEDY, request_id="mine")
    with pytest.raises(ValueError, match="already in use"):
        s.add_request([1], GREEDY, request_id="mine")
    tiny, _ = _make(num_pages=3, page=4, max_len=128)
    with pytest.raises(ValueError, match="does not fit the cache pool"):
        tiny.add_request(list(range(8)), GREEDY)


def test_prompt_is_cut_into_portions_and_sampled_with_the_last():
    s, ex = _make()
    r = s.add_request(list(range(37)), GREEDY)
    s.run_to_completion()
    # 16 + 16 + 5 (sampled), then three decode steps; the 4th token is never fed
    assert ex.steps == [[("req-0", 16, False)], [("req-0", 16, False)], [("req-0", 5, True)],
                        [("req-0", 1, True)], [("req-0", 1, True)], [("req-0", 1, True)]]
    assert r.output_token_ids == [1000, 1001, 1002, 1003] and r.finish_reason == "length"
    assert r.status is RequestStatus.FINISHED and not ex.cache.live_requests()


def test_decodes_run_beside_portions_under_one_budget():
    s, ex = _make(max_num_batched_tokens=20, max_chunk_size=16)
    rs = [s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=8))]
    s.step()  # a: whole prompt, sampled
    rs.append(s.add_request(list(range(40)), GREEDY))
    s.step()
    assert ex.steps[1] == [("req-0", 1, True), ("req-1", 16, False)]  # decode first, then the portion
    rs.append(s.add_request(list(range(30)), GREEDY))
    s.step()
    # budget 20: 1 decode + 16 of req-1 + 3 left for the newcomer's first portion
    assert ex.steps[2] == [("req-0", 1, True), ("req-1", 16, False), ("req-2", 3, False)]
    for shape in ex.steps:
        assert sum(n for _, n, _ in shape) <= 20
    s.run_to_completion()
    assert all(r.finish_reason == "length" for r in rs)
    assert not s._requests  # the engine keeps nothing of a finished request


def test_first_come_first_served_and_slot_limit():
    s, ex = _make(seqs=2)
    rs = [s.add_request([7] * 5, GREEDY) for _ in range(5)]
    s.step()
    assert [rid for rid, _, _ in ex.steps[0]] == ["req-0", "req-1"]  # two slots
    s.run_to_completion()
    first_step = {}
    for i, shape in enumerate(ex.steps):
        for rid, _, _ in shape:
            first_step.setdefault(rid, i)
    order = [first_step[r.request_id] for r in rs]
    assert order == sorted(order)  # nobody overtakes
    assert ex.cache.num_free_slots == 2
    for shape in ex.steps:
        assert len(shape) <= 2


def test_chunking_off_runs_whole_prompts_only():
    s, ex = _make(max_chunk_size=0, max_num_batched_tokens=128, max_len=128)
    s.add_request(list(range(100)), GREEDY)
    s.add_request(list(range(50)), GREEDY)
    s.step()
    assert ex.steps[0] == [("req-0", 100, True)]  # the second does not fit whole: it waits
    s.step()
    assert ex.steps[1] == [("req-0", 1, True), ("req-1", 50, True)]


def test_eos_is_not_counted_and_finishes():
    s, ex = _make(token=lambda rid, i: EOS if i == 2 else 5)
    r = s.add_request([1, 2], SamplingParams(temperature=0.0, max_gen_len=10))
    keep = s.add_request([1, 2], SamplingParams(temperature=0.0, max_gen_len=5, ignore_eos=True))
    s.run_to_completion()
    assert r.output_token_ids == [5, 5] and r.finish_reason == "eos"  # scheduler.py:1430-1436
    assert keep.output_token_ids == [5, 5, EOS, 5, 5] and keep.finish_reason == "length"


def test_length_cap_is_exact_at_the_context_limit():
    s, ex = _make(max_len=16)
    r = s.add_request(list(range(10)), SamplingParams(temperature=0.0))
    s.run_to_completion()
    assert len(r.output_token_ids) == 6 and r.seq_len == 16 and r.finish_reason == "length"
    assert ex.cache.num_free_pages() == 63


def test_abort_frees_everything():
    s, ex = _make()
    a = s.add_request(list(range(20)), GREEDY)
    b = s.add_request(list(range(20)), GREEDY)
    s.step()
    s.abort(a.request_id)
    s.abort(b.request_id)
    s.abort("nobody")
    assert a.finish_reason == b.finish_reason == "abort"
    assert not s.has_unfinished_requests() and not ex.cache.live_requests()
    ex.cache.check_invariants()


def test_when_pages_run_out_the_youngest_is_evicted_and_recomputed():
    # 7 usable pages of 4: two requests of 8 prompt tokens + 12 outputs need 5 pages each
    s, ex = _make(num_pages=8, page=4, token=lambda rid, i: (hash(rid) % 50) * 100 + i)
    params = SamplingParams(temperature=0.0, max_gen_len=12)
    a = s.add_request(list(range(8)), params)
    b = s.add_request(list(range(50, 58)), params)
    steps = 0
    while s.has_unfinished_requests():
        s.step()
        steps += 1
        assert steps < 200, "livelock"
    assert s.num_preemptions >= 1 and b.num_preemptions >= 1 and a.num_preemptions == 0
    for r in (a, b):
        base = (hash(r.request_id) % 50) * 100
        assert r.output_token_ids == [base + i for i in range(12)]  # nothing lost, nothing doubled
        assert r.finish_reason == "length"
    # the evicted request ran its own outputs again as if they were prompt
    evictions = [i for i, shape in enumerate(ex.steps) if any(rid == "req-1" and n > 1 for rid, n, _ in shape)]
    assert len(evictions) >= 2
    assert ex.cache.num_free_pages() == 7 and ex.cache.num_free_slots == 4
    ex.cache.check_invariants()


def test_evicted_request_returns_to_the_front_of_the_queue():
    s, ex = _make(num_pages=8, page=4, seqs=4)
    params = SamplingParams(temperature=0.0, max_gen_len=12)
    a = s.add_request(list(range(8)), params)
    b = s.add_request(list(range(8)), params)
    while s.num_preemptions == 0:
        s.step()
    late = s.add_request([1, 2, 3], params)
    assert s.waiting[0] is b and s.waiting[1] is late  # batch_planner.py:987-1023
    s.run_to_completion()
    assert len(b.output_token_ids) == 12 and len(late.output_token_ids) == 12


def test_a_request_alone_in_a_pool_too_small_ends_with_length():
    s, ex = _make(num_pages=4, page=4)  # 12 positions
    r = s.add_request(list(range(6)), SamplingParams(temperature=0.0, max_gen_len=50))
    s.run_to_completion()
    assert r.finish_reason == "length" and r.seq_len == 13  # the 13th token had no page to be fed into
    assert ex.cache.num_free_pages() == 3


def test_requests_stuck_in_their_prompts_do_not_deadlock():
    # both prompts fit alone but not together: neither can grow, nobody decodes
    s, ex = _make(num_pages=11, page=4, max_chunk_size=8, max_num_batched_tokens=16)
    params = SamplingParams(temperature=0.0, max_gen_len=2)
    a = s.add_request(list(range(36)), params)
    b = s.add_request(list(range(36)), params)
    steps = 0
    while s.has_unfinished_requests():
        s.step()
        steps += 1
        assert steps < 100
    assert len(a.output_token_ids) == 2 and len(b.output_token_ids) == 2
    assert b.num_preemptions >= 1 and a.num_preemptions == 0
    ex.cache.check_invariants()


def test_slot_and_page_conservation_over_many_rounds():
    import random

    rng = random.Random(3)
    s, ex = _make(num_pages=20, page=4, seqs=3, max_num_batched_tokens=24, max_chunk_size=8)
    done = []
    for round_ in range(30):
        for _ in range(rng.randrange(0, 3)):
            n = rng.randrange(1, 30)
            done.append(s.add_request([rng.randrange(90) for _ in range(n)],
                                      SamplingParams(temperature=0.0, max_gen_len=rng.randrange(1, 20))))
        for _ in range(rng.randrange(1, 6)):
            s.step()
            assert len(s.running) <= 3
    s.run_to_completion()
    assert all(r.is_finished and len(r.output_token_ids) == r.max_new_tokens for r in done)
    assert ex.cache.num_free_pages() == 19 and ex.cache.num_free_slots == 3
    # what was fed is the request's own sequence, in order (checked while it was live)


def test_fed_tokens_are_the_requests_own_sequence():
    s, ex = _make(num_pages=8, page=4, token=lambda rid, i: 200 + i)
    a = s.add_request(list(range(10)), SamplingParams(temperature=0.0, max_gen_len=9))
    b = s.add_request(list(range(30, 40)), SamplingParams(temperature=0.0, max_gen_len=9))
    while s.has_unfinished_requests():
        s.step()
        for r in s.running:
            fed = ex.fed.get(r.request_id, [])
            whole = r.prompt_token_ids + r.output_token_ids
            assert fed == whole[: len(fed)] and len(fed) == r.num_computed_tokens
    assert s.num_preemptions >= 1


def test_seeds_are_per_request_and_stable():
    s1, _ = _make(seed=5)
    s2, _ = _make(seed=5)
    s3, _ = _make(seed=6)
    a = [s1.add_request([1], GREEDY).seed for _ in range(3)]
    b = [s2.add_request([1], GREEDY).seed for _ in range(3)]
    c = [s3.add_request([1], GREEDY).seed for _ in range(3)]
    assert a == b and len(set(a)) == 3 and a != c
    assert s1.add_request([1], SamplingParams(seed=77)).seed == 77


def test_logprobs_are_collected_when_asked():
    s, _ = _make()
    r = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=3, logprobs=0))
    q = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=3))
    w = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=3, logprobs=2))
    s.run_to_completion()
    assert [x.logprob for x in r.output_logprobs] == [-1.0] * 3 and q.output_logprobs is None
    assert [x.token_id for x in r.output_logprobs] == r.output_token_ids
    assert all(x.top_token_ids == () for x in r.output_logprobs)
    assert [x.token_id for x in w.output_logprobs] == w.output_token_ids
    assert all(x.top_token_ids == (0, 1) and x.top_logprobs == (-2.0, -2.0) for x in w.output_logprobs)


def test_a_stop_token_leaves_no_record():
    s, _ = _make(token=lambda rid, i: EOS if i == 2 else 7)
    r = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=8, logprobs=1))
    s.run_to_completion()
    assert r.finish_reason == "eos" and r.output_token_ids == [7, 7] and len(r.output_logprobs) == 2


def test_prompt_logprobs_cover_every_position_once_across_portions():
    """Position q is scored by the logits at q - 1, whichever portion holds them: the last
    place of a portion scores the first token of the next one; position 0 has no predictor
    (rapid_llm/engine/scheduler.py:143-148, rapid_llm/engine/llm_engine.py:274-291)."""
    s, ex = _make(max_chunk_size=4, max_num_batched_tokens=6)
    prompt = list(range(20, 31))  # 11 tokens: portions of 4, 4, 3
    r = s.add_request(prompt, SamplingParams(temperature=0.0, max_gen_len=3, prompt_logprobs=2, logprobs=0))
    other = s.add_request([5, 6, 7, 8, 9], SamplingParams(temperature=0.0, max_gen_len=3))
    s.run_to_completion()
    assert other.prompt_logprobs is None
    assert len(r.prompt_logprobs) == 11 and r.prompt_logprobs[0] is None
    assert [x.token_id for x in r.prompt_logprobs[1:]] == prompt[1:]
    assert all(x.top_token_ids == (0, 1) for x in r.prompt_logprobs[1:])
    mine = [(start, want) for rid, start, _, want in ex.wants if rid == r.request_id]
    # every place of a portion but the prompt's last is scored; the last one chooses a token
    assert mine[:3] == [(0, [0, 1, 2, 3]), (4, [0, 1, 2, 3]), (8, [0, 1, 2])]
    assert all(want == [0] for _, want in mine[3:])
    assert len(r.output_logprobs) == 3


def test_prompt_logprobs_of_one_token_prompt_and_after_eviction():
    s, _ = _make()
    r = s.add_request([4], SamplingParams(temperature=0.0, max_gen_len=2, prompt_logprobs=0))
    s.run_to_completion()
    assert r.prompt_logprobs == [None]
    # a pool of 6 pages of 4: two requests outgrow it, one is evicted and runs again; what
    # was scored before the eviction is kept and not asked for again
    s, ex = _make(num_pages=7, page=4, seqs=2, max_len=64)
    params = SamplingParams(temperature=0.0, max_gen_len=12, prompt_logprobs=1)
    a = s.add_request(list(range(10, 16)), params)
    b = s.add_request(list(range(30, 36)), params)
    s.run_to_completion()
    assert s.num_preemptions > 0
    for r in (a, b):
        assert [x.token_id for x in r.prompt_logprobs[1:]] == r.prompt_token_ids[1:]
    evicted = a if a.num_preemptions else b
    again = [(n, want) for rid, start, n, want in ex.wants if rid == evicted.request_id and start == 0]
    assert again[0] == (6, [0, 1, 2, 3, 4, 5]) and len(again) >= 2
    assert all(want == [n - 1] for n, want in again[1:])


def test_repetition_breaker():
    assert not detect_repetition(list(range(200)))
    loop = list(range(32)) * 5
    assert detect_repetition(loop)
    assert not detect_repetition(loop[:100])
    s, _ = _make(max_len=512, num_pages=200, token=lambda rid, i: i % 8)
    r = s.add_request([1], SamplingParams(temperature=0.0, stop_on_repeat=True))
    free = s.add_request([1], SamplingParams(temperature=0.0, max_gen_len=300))
    s.run_to_completion()
    assert r.finish_reason == "repeat" and len(r.output_token_ids) < 200
    assert free.finish_reason == "length" and len(free.output_token_ids) == 300


def test_sampling_params_validation():
    SamplingParams()
    for bad in (dict(temperature=-1), dict(top_p=0), dict(top_p=1.5), dict(max_gen_len=0),
                dict(repetition_penalty=0), dict(logprobs=-1), dict(prompt_logprobs=-1),
                dict(seed=-3)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
    assert SamplingParams(temperature=0).is_greedy and not SamplingParams().is_greedy


# ------------------------------------------------------------------ the launch/harvest pipeline
def _workload(scheduler, seed, n=9, penalty=False):
    import random

    rng = random.Random(seed)
    requests = []
    for i in range(n):
        prompt = [rng.randrange(50) for _ in range(rng.choice([1, 2, 5, 17, 30]))]
        params = SamplingParams(
            temperature=0.0, max_gen_len=rng.choice([1, 2, 3, 9, 24]),
            repetition_penalty=1.3 if penalty and i % 3 == 0 else 1.0,
            stop_on_repeat=i % 4 == 0, logprobs=0 if i % 2 else None,
            prompt_logprobs=1 if i % 5 == 0 else None,
        )
        requests.append(scheduler.add_request(prompt, params))
    return requests


def _token_with_stops(rid, i):
    # some requests meet a stop token early, some late, some never
    n = int(rid.split("-")[1])
    return EOS if (n % 3 == 1 and i == 2 + n % 5) else (n * 31 + i * 7) % 50


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("pool", [200, 21, 13])
def test_pipeline_changes_no_token(seed, pool):
    """Queueing step N + 1 before step N is read gives every request the tokens, the finish
    reason and the records of the synchronous loop: ample pages, and pools so small that
    requests are evicted (the schedules then differ, the results must not)."""
    outcomes = []
    for pipeline in (False, True):
        s, ex = _make_pipelined(num_pages=pool, page=4, seqs=3, max_len=64, token=_token_with_stops,
                                pipeline=pipeline, max_num_batched_tokens=24, max_chunk_size=8)
        requests = _workload(s, seed)
        steps = 0
        while s.has_unfinished_requests():
            s.step()
            steps += 1
            assert steps < 2000
        assert ex.max_unread == (2 if pipeline else 1)
        assert not ex.cache.live_requests() and not s._held and ex.unread == 0
        ex.cache.check_invariants()
        outcomes.append([
            (r.output_token_ids, r.finish_reason,
             None if r.output_logprobs is None else [x.token_id for x in r.output_logprobs],
             None if r.prompt_logprobs is None else [x and x.token_id for x in r.prompt_logprobs])
            for r in requests
        ])
        assert all(r.pending == 0 and r.discard == 0 for r in requests)
    assert outcomes[0] == outcomes[1]


def test_pipeline_feeds_tokens_from_the_device_and_stops_one_step_late():
    s, ex = _make_pipelined(token=lambda rid, i: EOS if i == 3 else 40 + i)
    r = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=10))
    while s.has_unfinished_requests():
        s.step()
    assert r.output_token_ids == [40, 41, 42] and r.finish_reason == "eos"
    # prompt, then one decoded token a step; the step after the stop token ran and was dropped
    assert [shape for shape in ex.steps] == [[(r.request_id, 3, True)]] + [[(r.request_id, 1, True)]] * 4
    assert not ex.cache.live_requests()


def test_pipeline_ends_by_count_cost_no_extra_step():
    s, ex = _make_pipelined()
    r = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=4))
    while s.has_unfinished_requests():
        s.step()
    assert len(r.output_token_ids) == 4 and r.finish_reason == "length"
    assert len(ex.steps) == 4  # the prompt's step chooses the first token, three decodes the rest
    s, ex = _make_pipelined(max_len=8)
    r = s.add_request([1, 2, 3, 4, 5], SamplingParams(temperature=0.0))
    while s.has_unfinished_requests():
        s.step()
    assert r.seq_len == 8 and r.finish_reason == "length" and len(ex.steps) == 3


@pytest.mark.parametrize("seed", range(4))
@pytest.mark.parametrize("pool", [200, 17])
def test_a_penalty_rides_the_pipeline(seed, pool):
    """A penalised request's history names the token still on the device by its sampling row;
    the tokens, which depend on the whole history, are those of the synchronous loop."""
    outcomes = []
    for pipeline in (False, True):
        s, ex = _make_pipelined(num_pages=pool, pipeline=pipeline, seqs=3, max_len=64, token=_token_with_stops,
                                max_num_batched_tokens=24, max_chunk_size=8)
        requests = _workload(s, seed, penalty=True)
        while s.has_unfinished_requests():
            s.step()
        assert ex.max_unread == (2 if pipeline else 1)
        outcomes.append([(r.output_token_ids, r.finish_reason) for r in requests])
        assert not ex.cache.live_requests()
    assert outcomes[0] == outcomes[1]
    assert any(len(set(out)) == len(out) > 8 for out, _ in outcomes[0]), "no penalised request ran long"


def test_abort_while_a_step_is_in_flight():
    s, ex = _make_pipelined()
    r = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=10))
    q = s.add_request([4, 5], SamplingParams(temperature=0.0, max_gen_len=3))
    s.step()
    s.step()
    assert r.pending == 1
    s.abort(r.request_id)
    assert r.finish_reason == "abort" and ex.cache.has(r.request_id)  # held until the step is read
    kept = list(r.output_token_ids)
    while s.has_unfinished_requests():
        s.step()
    assert r.output_token_ids == kept and not ex.cache.live_requests()
    assert len(q.output_token_ids) == 3


@pytest.mark.parametrize("pipeline", [True, False])
def test_an_id_is_used_again_while_its_last_step_is_still_in_flight(pipeline):
    """A request that a stop token ended rides one more step, on whose slot and pages it is
    still held; the same id submitted at that moment names a new request, which waits that one
    step and then runs as any other."""
    s, ex = _make_pipelined(token=lambda rid, i: EOS if i == 1 else 40 + i, pipeline=pipeline)
    first = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=10), request_id="x")
    while not first.is_finished:
        s.step()
    assert first.finish_reason == "eos" and first.output_token_ids == [40]
    if pipeline:
        assert [r.request_id for r in s._held] == ["x"] and ex.cache.has("x")
    second = s.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_gen_len=10), request_id="x")
    assert second is not first
    other = s.add_request([5, 6], SamplingParams(temperature=0.0, max_gen_len=3))
    steps = 0
    while s.has_unfinished_requests():
        s.step()
        steps += 1
        assert steps < 50
    assert second.finish_reason == "eos" and second.output_token_ids == [40]
    assert first.output_token_ids == [40] and first.pending == 0 and first.discard == 0
    assert len(other.output_token_ids) == 1 and other.finish_reason == "eos"
    assert not ex.cache.live_requests() and not s._held and not s._requests
    ex.cache.check_invariants()
    with pytest.raises(ValueError, match="already in use"):
        s.add_request([1], GREEDY, request_id="y")
        s.add_request([1], GREEDY, request_id="y")


def test_request_tokens_name_the_pending_row():
    s, ex = _make_pipelined()
    r = s.add_request([7, 8, 9], SamplingParams(temperature=0.0, max_gen_len=5))
    s.step()
    assert r.pending == 1 and r.seq_len == 4 and r.tokens(2, 4) == [9, fed_token(0)]
    s.step()  # queues the decode of the fed token, then reads the first token
    assert r.output_token_ids == [1000] and r.pending == 1 and r.tokens(0, 5) == [7, 8, 9, 1000, fed_token(0)]
