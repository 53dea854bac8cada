"""The sampling kernels against the plain sampler: arg-max, temperature, nucleus with its
pool of 1024, repetition penalty, seeded draws; at vocabularies from 3 to 151,936."""

import pytest
import torch

from plain_sampler import plain_logprob, plain_sample
from rapid_llm_amd.sampling.rng import uniform_draw

pytestmark = pytest.mark.gpu


def _sampler():
    from rapid_llm_amd.sampling.sampler import RowSampling, Sampler

    return Sampler("cuda"), RowSampling


def _acceptable(logits, row, u):
    """Tokens the plain sampler picks for draws within rounding of ``u``: the kernel sums
    its probabilities in float32 in another order."""
    return {
        plain_sample(logits, row.temperature, row.top_p, min(max(u + d, 0.0), 0.9999999),
                     row.repetition_penalty, list(row.generated))
        for d in (0.0, -3e-6, 3e-6)
    }


def test_uniform_draw_matches_the_kernel():
    from rapid_llm_amd.kernels import ops

    for seed, counter in [(0, 0), (1, 0), (0, 1), (2**63 + 12345, 99), (2**64 - 1, 2**32 - 1)]:
        assert ops.sample_uniform(seed, counter) == uniform_draw(seed, counter)
    draws = [uniform_draw(42, i) for i in range(4000)]
    assert 0.0 <= min(draws) and max(draws) < 1.0 and abs(sum(draws) / 4000 - 0.5) < 0.02


@pytest.mark.parametrize("vocab", [3, 64, 503, 1024, 1025, 4099, 151936])
def test_rows_of_every_kind_match_the_plain_sampler(vocab):
    sampler, Row = _sampler()
    gen = torch.Generator().manual_seed(vocab)
    rows, logit_rows = [], []
    kinds = [
        dict(temperature=0.0, top_p=1.0),
        dict(temperature=0.0, top_p=0.9, repetition_penalty=1.3),
        dict(temperature=0.8, top_p=1.0),
        dict(temperature=0.8, top_p=0.9),
        dict(temperature=1.5, top_p=0.5, repetition_penalty=1.2),
        dict(temperature=0.3, top_p=0.1),
        dict(temperature=2.5, top_p=0.999),
        dict(temperature=1.0, top_p=0.95, repetition_penalty=0.8),
    ]
    for i in range(24):
        kind = kinds[i % len(kinds)]
        scale = (1.0, 4.0, 0.2)[i % 3]
        logit_rows.append(torch.randn(vocab, generator=gen) * scale)
        generated = torch.randint(0, vocab, (17,), generator=gen).tolist() + [int(logit_rows[-1].argmax())]
        rows.append(Row(seed=1000 + i, counter=i * 7, generated=generated, **kind))
    logits = torch.stack(logit_rows).cuda()
    ids, logprobs = sampler.sample(logits, rows, want_logprobs=True)
    ids, logprobs = ids.tolist(), logprobs.tolist()
    for i, row in enumerate(rows):
        u = uniform_draw(row.seed, row.counter)
        assert ids[i] in _acceptable(logit_rows[i], row, u), (vocab, i, row)
        want = plain_logprob(logit_rows[i], ids[i], row.temperature, row.repetition_penalty, list(row.generated))
        assert abs(logprobs[i] - want) < 2e-4 * max(1.0, abs(want)), (vocab, i)


def test_greedy_batch_takes_the_argmax_kernel_and_lowest_index_wins():
    sampler, Row = _sampler()
    logits = torch.randn(9, 7001)
    logits[3, 100] = logits[3, 4000] = 50.0  # equal maxima: the lower index
    logits[5, :] = 1.25
    ids, lp = sampler.sample(logits.cuda(), [Row() for _ in range(9)])
    assert lp is None
    want = logits.argmax(-1).tolist()
    want[3], want[5] = 100, 0
    assert ids.tolist() == want
    # the general kernel's greedy rows agree
    ids2, _ = sampler.sample(logits.cuda(), [Row() for _ in range(9)], want_logprobs=True)
    assert ids2.tolist() == want


def test_reference_vectors():
    sampler, Row = _sampler()
    # rapid_llm tests/engine/test_sampler.py:61-63
    ids, _ = sampler.sample(torch.tensor([[0.1, 0.9, 0.0], [0.5, 0.1, 0.4]]).cuda(), [Row(), Row()])
    assert ids.tolist() == [1, 0]
    # :66-72 a nucleus of 0.1 keeps only the dominant token, whatever the draw
    logits = torch.log(torch.tensor([[0.7, 0.2, 0.1]])).cuda().repeat(64, 1)
    ids, _ = sampler.sample(logits, [Row(temperature=1.0, top_p=0.1, seed=5, counter=c) for c in range(64)])
    assert set(ids.tolist()) == {0}
    # :229-266 the penalty divides positive and multiplies negative logits, once per token
    logits = torch.tensor([[4.0, -4.0, 3.9], [4.0, 3.0, -9.0]]).cuda()
    ids, _ = sampler.sample(logits, [Row(repetition_penalty=2.0, generated=[0, 0, 1]),
                                     Row(repetition_penalty=1.2, generated=[0, 0, 0, 0])])
    assert ids.tolist() == [2, 0]  # row 0: 4/2 < 3.9; row 1: 4/1.2 = 3.33 > 3 (applied once, not four times)


def test_draws_follow_the_distribution_and_the_seed():
    sampler, Row = _sampler()
    probs = torch.tensor([0.05, 0.5, 0.25, 0.2])
    n = 4096
    logits = torch.log(probs)[None].repeat(n, 1).cuda()
    for top_p, want in ((1.0, probs), (0.8, torch.tensor([0.0, 0.5, 0.25, 0.2]) / 0.95)):
        ids, _ = sampler.sample(logits, [Row(temperature=1.0, top_p=top_p, seed=9, counter=c) for c in range(n)])
        freq = torch.bincount(ids.cpu().long(), minlength=4).float() / n
        assert float((freq - want).abs().max()) < 0.03, (top_p, freq)
        again, _ = sampler.sample(logits, [Row(temperature=1.0, top_p=top_p, seed=9, counter=c) for c in range(n)])
        assert torch.equal(ids, again)
        other, _ = sampler.sample(logits, [Row(temperature=1.0, top_p=top_p, seed=10, counter=c) for c in range(n)])
        assert not torch.equal(ids, other)


def test_pool_never_leaks_and_flat_rows_keep_the_whole_pool():
    sampler, Row = _sampler()
    vocab = 5000
    flat = torch.zeros(256, vocab).cuda()  # more equal logits than the pool has places
    ids, _ = sampler.sample(flat, [Row(temperature=1.0, top_p=0.999, seed=3, counter=c) for c in range(256)])
    assert max(ids.tolist()) < 1024 and len(set(ids.tolist())) > 100  # the lowest indices fill the pool
    gen = torch.Generator().manual_seed(0)
    logits = torch.randn(64, vocab, generator=gen) * 0.01  # nearly flat: the pool never reaches top_p
    pool = [set(r.topk(1024).indices.tolist()) for r in logits]
    ids, _ = sampler.sample(logits.cuda(), [Row(temperature=1.0, top_p=0.9, seed=4, counter=c) for c in range(64)])
    assert all(t in pool[i] for i, t in enumerate(ids.tolist()))


def test_penalty_needs_a_vocabulary_the_bitmap_holds():
    from rapid_llm_amd.kernels.ops import KernelError

    sampler, Row = _sampler()
    logits = torch.zeros(1, 400_000).cuda()
    sampler.sample(logits, [Row(temperature=1.0, top_p=0.9)])  # no penalty: fine
    with pytest.raises(KernelError, match="beyond"):
        sampler.sample(logits, [Row(temperature=1.0, repetition_penalty=1.1, generated=[1])])


@pytest.mark.parametrize("vocab", [3, 64, 503, 4099, 151936])
def test_logprob_records_match_the_plain_ones(vocab):
    """The given token's log-probability and the k most likely, under the distribution the
    row is sampled from (penalty, temperature, greedy as temperature 1) and under the raw
    logits; rows read through an index, in another order than they lie."""
    from plain_sampler import plain_top_logprobs

    sampler, Row = _sampler()
    gen = torch.Generator().manual_seed(7 * vocab)
    kinds = [dict(temperature=0.0), dict(temperature=0.7), dict(temperature=1.6, repetition_penalty=1.4),
             dict(temperature=0.0, repetition_penalty=0.7)]
    n = 9
    logit_rows = [torch.randn(vocab, generator=gen) * (1.0, 5.0, 0.3)[i % 3] for i in range(n)]
    # equal values: the lower id comes first, among the best and further down
    logit_rows[2][: min(vocab, 6)] = float(logit_rows[2].max()) + 1.0
    logit_rows[4][vocab // 2 :] = -3.0
    order = [5, 0, 8, 2, 4, 7, 1]
    rows, targets = [], []
    for b, r in enumerate(order):
        generated = torch.randint(0, vocab, (11,), generator=gen).tolist() + [int(logit_rows[r].argmax())]
        rows.append(Row(seed=b, counter=b, generated=generated, **kinds[b % len(kinds)]))
        targets.append(int(torch.randint(0, vocab, (1,), generator=gen)))
    logits = torch.stack(logit_rows).cuda()
    k = min(vocab, 7)
    for with_rows in (True, False):
        target_lp, top_ids, top_lp = sampler.logprobs(
            logits, targets, k, rows=rows if with_rows else None, row_index=order)
        target_lp, top_ids, top_lp = target_lp.tolist(), top_ids.tolist(), top_lp.tolist()
        for b, r in enumerate(order):
            row = rows[b] if with_rows else Row(temperature=1.0)
            args = (row.temperature, row.repetition_penalty, list(row.generated))
            want = plain_logprob(logit_rows[r], targets[b], *args)
            assert abs(target_lp[b] - want) < 2e-4 * max(1.0, abs(want)), (vocab, b)
            ids, lps = plain_top_logprobs(logit_rows[r], k, *args)
            assert top_ids[b] == ids, (vocab, with_rows, b)
            assert max(abs(x - y) for x, y in zip(top_lp[b], lps)) < 2e-4 * max(1.0, abs(lps[-1])), (vocab, b)
    # k = 0: the token's own log-probability only; without an index the rows in order
    lp0, ids0, _ = sampler.logprobs(logits, [1] * n, 0)
    assert ids0.shape == (n, 0)
    for r in range(n):
        want = plain_logprob(logit_rows[r], 1, 1.0)
        assert abs(float(lp0[r]) - want) < 2e-4 * max(1.0, abs(want))


def test_logprob_records_with_values_that_cannot_be_ordered():
    """NaN is never listed: with fewer than k comparable values the rest is marked empty;
    -inf is comparable and comes last, by ascending id."""
    sampler, _ = _sampler()
    logits = torch.tensor([[0.5, float("nan"), -float("inf"), 2.0, -float("inf")]]).cuda()
    _, ids, _ = sampler.logprobs(logits, [3], 5)
    assert ids.tolist() == [[3, 0, 2, 4, -1]]
    logits = torch.tensor([[0.5, -float("inf"), 2.0, -float("inf")]]).cuda()
    lp, ids, lps = sampler.logprobs(logits, [1], 4)
    assert ids.tolist() == [[2, 0, 1, 3]] and lp.item() == -float("inf")
    assert lps[0, 2:].tolist() == [-float("inf")] * 2 and abs(lps[0, :2].exp().sum().item() - 1.0) < 1e-6


def test_sampling_through_a_row_index():
    sampler, Row = _sampler()
    gen = torch.Generator().manual_seed(5)
    logits = torch.randn(12, 9001, generator=gen).cuda()
    index = [11, 3, 3, 0, 7]
    ids, _ = sampler.sample(logits, [Row() for _ in index], row_index=index)
    assert ids.tolist() == logits.argmax(-1)[index].tolist()
    rows = [Row(temperature=0.9, top_p=0.8, seed=3, counter=i) for i in range(len(index))]
    picked, _ = sampler.sample(logits, rows, row_index=index)
    direct, _ = sampler.sample(logits[index].contiguous(), rows)
    assert picked.tolist() == direct.tolist()


def test_a_history_may_name_tokens_still_on_the_device():
    """A history entry -(r + 1) is read as row r of the choices of the step before: the chosen
    tokens and the records are those of the history written out; a row beyond that buffer and
    a buffer that this call overwrites are refused."""
    from rapid_llm_amd.kernels.ops import KernelError

    sampler, Row = _sampler()
    gen = torch.Generator().manual_seed(11)
    vocab = 5003
    logits = (torch.randn(4, vocab, generator=gen) * 0.05)
    before = [17, 4000, 2, 911, 77]  # what five rows of the step before chose
    for i, tok in enumerate(before[:4]):
        logits[i, tok] = 6.0  # without the penalty each row would choose its own newest token
        logits[i, 100 + i] = 5.0  # with it, the runner-up
    logits = logits.cuda()
    fed = torch.tensor(before, dtype=torch.int32, device="cuda")
    named = [[30, 31, -3], [-2], [5, 6, 7, 8, -1], [-4]]
    written = [[30, 31, before[2]], [before[1]], [5, 6, 7, 8, before[0]], [before[3]]]
    index = [2, 1, 0, 3]  # sampling row b reads the logits row whose favourite its history names
    kinds = [dict(temperature=0.0), dict(temperature=0.7, top_p=0.9, seed=5, counter=3),
             dict(temperature=0.0), dict(temperature=1.3, seed=9, counter=1)]
    rows_named = [Row(repetition_penalty=4.0, generated=g, **k) for g, k in zip(named, kinds)]
    rows_written = [Row(repetition_penalty=4.0, generated=g, **k) for g, k in zip(written, kinds)]
    got, got_lp = sampler.sample(logits, rows_named, want_logprobs=True, row_index=index, fed=fed)
    want, want_lp = sampler.sample(logits, rows_written, want_logprobs=True, row_index=index)
    assert got.tolist() == want.tolist()
    assert got.tolist()[0] == 102 and got.tolist()[2] == 100  # the greedy rows: the runner-up
    assert torch.equal(got_lp, want_lp)
    a = sampler.logprobs(logits, got, 3, rows=rows_named, row_index=index, fed=fed)
    b = sampler.logprobs(logits, want, 3, rows=rows_written, row_index=index)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    with pytest.raises(ValueError, match="names sampling row 5"):
        sampler.sample(logits, [Row(repetition_penalty=2.0, generated=[-6])] * 4, fed=fed)
    with pytest.raises(ValueError, match="names sampling row 0"):
        sampler.sample(logits, [Row(repetition_penalty=2.0, generated=[-1])] * 4)
    with pytest.raises(KernelError, match="share memory"):
        sampler.sample(logits, rows_named, row_index=index, out=fed, fed=fed)
