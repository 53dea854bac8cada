"""Each HIP kernel alone against its plain reference, at sizes other than the tiny models'."""

import math
import random
from types import SimpleNamespace

import pytest
import torch

from plain_model import plain_attention, plain_inv_freq, plain_rmsnorm, plain_rope_apply, plain_rope_tables
from rotation_reference import rotate_pairs

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ops():
    from rapid_llm_amd.kernels import ops

    return ops


# --------------------------------------------------------------------------- #
# a paged cache laid out by hand: pages in shuffled order, everything else NaN
# --------------------------------------------------------------------------- #
def _paged_problem(seqs, nq, nkv, d, page, dtype, seed, window=0, spike=None):
    """``seqs`` = list of (tokens already cached, tokens in this step).  Returns the kernel
    operands and the expected output from the plain attention."""
    rng = random.Random(seed)
    gen = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(a + n) // page) for a, n in seqs) + 1
    order = list(range(1, total_pages))
    rng.shuffle(order)
    max_pages = max(-(-(a + n) // page) for a, n in seqs) + 2
    table = torch.zeros((len(seqs) + 3, max_pages), dtype=torch.int32)
    k_cache = torch.full((total_pages, nkv, page, d), float("nan"))
    v_cache = torch.full((total_pages, nkv, d, page), float("nan"))
    slots = list(range(len(seqs) + 3))
    rng.shuffle(slots)
    q_rows, positions, token_slot, expect = [], [], [], []
    for i, (a, n) in enumerate(seqs):
        t = a + n
        k = torch.randn((t, nkv, d), generator=gen)
        v = torch.randn((t, nkv, d), generator=gen)
        q = torch.randn((n, nq, d), generator=gen)
        if spike is not None and i == spike[0]:
            # one far key carries nearly all of the softmax mass of the last query
            far = spike[1]
            group = nq // nkv
            for j in range(nkv):
                u = q[-1, j * group].clone()
                q[-1, j * group : (j + 1) * group] = u  # the heads of a group ask alike
                k[far, j] = u * (30.0 * math.sqrt(d) / float(u @ u))  # score 30 against ~N(0,1)
            v[far] = 7.0
        if dtype == torch.bfloat16:
            q, k, v = (x.bfloat16().float() for x in (q, k, v))
        slot = slots[i]
        for p in range(-(-t // page)):
            pid = order.pop()
            table[slot, p] = pid
            lo, hi = p * page, min(t, (p + 1) * page)
            k_cache[pid, :, : hi - lo, :] = k[lo:hi].transpose(0, 1)
            v_cache[pid, :, :, : hi - lo] = v[lo:hi].permute(1, 2, 0)
        qpos = torch.arange(a, t)
        expect.append(
            plain_attention(q, k, v, 1.0 / math.sqrt(d), window or None, qpos, torch.arange(t)).reshape(n, nq * d)
        )
        q_rows.append(q.reshape(n, nq * d))
        positions += list(range(a, t))
        token_slot += [slot] * n
    ctx = SimpleNamespace(
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
        token_slot=torch.tensor(token_slot, dtype=torch.int32, device=DEV),
        token_ids=torch.zeros(len(positions), dtype=torch.int32, device=DEV),
        h_seq_starts=[a for a, _ in seqs],
        h_seq_lens=[n for _, n in seqs],
        max_position=max(positions),
        extra={},
    )
    return (
        torch.cat(q_rows).to(DEV, dtype),
        k_cache.to(DEV, dtype),
        v_cache.to(DEV, dtype),
        table.to(DEV),
        ctx,
        torch.cat(expect),
    )


ATTN_CASES = [
    # nq, nkv, d, page, window, seqs
    (7, 7, 16, 4, 0, [(0, 5), (37, 1), (3, 2)]),
    (12, 3, 48, 8, 0, [(0, 130), (200, 1), (64, 33), (0, 1)]),
    (20, 1, 80, 16, 0, [(300, 1), (5, 70), (0, 2)]),          # 20 heads on one kv head
    (8, 2, 128, 16, 0, [(700, 1), (0, 257), (511, 1), (100, 29)]),
    (4, 4, 256, 32, 0, [(90, 1), (0, 75)]),
    (6, 2, 64, 4, 19, [(0, 90), (45, 1), (200, 1), (30, 31)]),  # window
    (10, 5, 112, 12, 40, [(333, 1), (77, 50)]),
    (8, 2, 128, 16, 0, [(20000, 1), (16000, 150), (9000, 1)]),  # long contexts: many splits, a long prefix
    (4, 1, 64, 8, 3000, [(12000, 1), (5000, 40)]),               # a window deep in a long context
    (8, 2, 128, 16, 0, [(3584, 512)]),   # one portion of a long prompt: few, long tiles, their keys cut into runs
    (6, 3, 64, 8, 0, [(1500, 300), (40, 1), (2100, 33)]),  # the same beside a single token, odd lengths
    # the head counts of the family's two larger dense models (groups of 8 and of 5 query heads a
    # kv head): a single token over 9,000 keys, a portion of 512 behind 7,000, a two-token portion
    (64, 8, 128, 16, 0, [(9000, 1), (7000, 512), (5, 2)]),
    (40, 8, 128, 16, 0, [(9001, 1), (6990, 512), (0, 2)]),
]


# bfloat16 attention against the plain attention of the same bfloat16 operands: the worst element's
# error and the worst row's rms error, relative to the spread of that request's outputs (the
# mean of many values shrinks with the number of keys, and an absolute bound would grow lax with
# it).  What is left is the rounding of the softmax weights and of the result: worst seen 0.036
# (a prompt from its start: the first rows are single values, far larger than the spread of all
# rows) and 0.0069.
BF16_ATTN_PEAK = 0.06
BF16_ATTN_ROW = 0.012


def _close_bf16_attention(got, want, seqs, label=""):
    at = 0
    for a, n in seqs:
        g, w = got[at : at + n].double(), want[at : at + n].double()
        at += n
        spread = float(w.std())
        peak = float((g - w).abs().max()) / spread
        row = float((g - w).square().mean(dim=1).sqrt().max()) / spread
        print(f"attention {label} ({a}+{n}): peak {peak:.4f} row {row:.4f} of the outputs' spread {spread:.4f}")
        assert peak <= BF16_ATTN_PEAK and row <= BF16_ATTN_ROW, (label, a, n, peak, row)


@pytest.mark.parametrize("case", ATTN_CASES, ids=lambda c: f"h{c[0]}kv{c[1]}d{c[2]}p{c[3]}w{c[4]}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_paged_attention(case, dtype):
    ops = _ops()
    nq, nkv, d, page, window, seqs = case
    q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, dtype, seed=len(seqs) * 7 + d, window=window)
    out = torch.full_like(q, float("nan"))
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, window, 1.0 / math.sqrt(d))
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-5, atol=2e-6)
    else:
        _close_bf16_attention(got, want, seqs, "paged")


def test_order_by_length_names_the_longest_first():
    """The order the decode attention hands its workgroups out in: the requests' indices by
    descending last position, equal ones in their own order; with and without a list of the
    requests' tokens, at sizes around the kernel's blocks of 256."""
    import ctypes

    ops = _ops()
    core = ops.core()
    gen = torch.Generator().manual_seed(5)
    for n, spread in [(1, 10), (7, 3), (256, 40), (257, 100000), (700, 5)]:
        lengths = torch.randint(0, spread, (n,), generator=gen, dtype=torch.int32)
        want = sorted(range(n), key=lambda i: (-int(lengths[i]), i))
        # (a) request i is token i
        order = torch.full((n,), -1, dtype=torch.int32, device=DEV)
        dev_lengths = lengths.to(DEV)
        rc = core.rl_order_by_length(ctypes.c_void_p(dev_lengths.data_ptr()), None, n,
                                     ctypes.c_void_p(order.data_ptr()), ops._stream())
        assert rc == 0 and order.cpu().tolist() == want, (n, spread)
        # (b) the requests' tokens lie scattered among others
        perm = torch.randperm(3 * n, generator=gen)[:n].to(torch.int32)
        positions = torch.full((3 * n,), 10**6, dtype=torch.int32)
        positions[perm.long()] = lengths
        order.fill_(-1)
        dev_positions, dev_tokens = positions.to(DEV), perm.to(DEV)
        rc = core.rl_order_by_length(ctypes.c_void_p(dev_positions.data_ptr()),
                                     ctypes.c_void_p(dev_tokens.data_ptr()), n,
                                     ctypes.c_void_p(order.data_ptr()), ops._stream())
        assert rc == 0 and order.cpu().tolist() == want, (n, spread, "scattered")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_decode_attention_of_many_requests_of_mixed_lengths(dtype):
    """More workgroups than the chip holds at a time: the decode kernel then takes the requests
    longest first, from an order made on the device, and every die a different head of each.
    260 single tokens over contexts of 1 to 700 keys beside two portions, 3 kv heads of 2 query
    heads; the request with the one-key context and the longest are both there."""
    ops = _ops()
    rng = random.Random(11)
    nq, nkv, d, page = 6, 3, 64, 8
    seqs = [(rng.randint(0, 699), 1) for _ in range(258)] + [(0, 1), (699, 1), (40, 9), (0, 3)]
    rng.shuffle(seqs)
    q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, dtype, seed=77)
    out = torch.full_like(q, float("nan"))
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, 0, 1.0 / math.sqrt(d))
    if dtype == torch.bfloat16:
        plan = ops.attention_plan(ctx, nq // nkv, d)
        assert plan.num_decode == 260 and plan.num_decode * nkv > ops.chip().decode_resident
        order = plan._decode_order
        assert order is not None, "the launch was not ordered"
        tokens = plan.seq_token.cpu().tolist()
        lengths = [int(ctx.positions[t]) for t in tokens]
        assert order.cpu().tolist() == sorted(range(260), key=lambda i: (-lengths[i], i))
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-5, atol=2e-6)
    else:
        _close_bf16_attention(got, want, seqs, "mixed lengths")


PREFILL_SHAPE_CASES = [
    # nq, nkv, d, page, window, seqs: portions only
    (8, 2, 128, 16, 0, [(0, 200), (700, 90), (0, 3)]),     # tiles of one step (the second wave group idle) and of many
    (6, 3, 64, 8, 0, [(130, 61), (1000, 130)]),            # odd numbers of steps
    (6, 2, 48, 4, 70, [(0, 300), (500, 40)]),              # a window: steps before it are never read
    (4, 4, 256, 32, 0, [(40, 100)]),                       # the largest tiles in LDS
    (5, 5, 16, 4, 0, [(0, 77), (90, 2)]),                  # the smallest
    # head size 128 with pages of a multiple of eight keys: tiles loaded straight into LDS, two
    # sets in turn; a window (the first and last steps of a tile are repaired in LDS), and
    # pages of four and twelve keys, which keep to the tiles staged through registers
    (8, 2, 128, 16, 150, [(0, 333), (900, 100), (40, 2)]),
    (4, 4, 128, 8, 0, [(0, 129), (260, 70)]),
    (8, 4, 128, 4, 0, [(100, 90), (0, 3)]),
    (6, 2, 128, 12, 50, [(30, 200)]),
]


@pytest.mark.parametrize("case", PREFILL_SHAPE_CASES, ids=lambda c: f"h{c[0]}kv{c[1]}d{c[2]}p{c[3]}w{c[4]}")
@pytest.mark.parametrize("shape", [(1, 1), (2, 1), (1, 3), (2, 3), (2, 8)], ids=lambda s: f"g{s[0]}n{s[1]}")
def test_prefill_attention_in_every_launch_shape(case, shape, monkeypatch):
    """One or two wave groups on a tile, its keys whole or cut into runs: the host picks by the
    launch's size, here every combination is forced on the same problems."""
    ops = _ops()
    monkeypatch.setattr(ops, "_prefill_shape", lambda *a, **k: shape)
    nq, nkv, d, page, window, seqs = case
    q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, torch.bfloat16, seed=d + page, window=window)
    out = torch.full_like(q, float("nan"))
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, window, 1.0 / math.sqrt(d))
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    _close_bf16_attention(got, want, seqs, f"prefill shape {shape}")


def test_prefill_shape_follows_the_launch():
    """Two wave groups where the longest tile would outlast everyone else's work (one prompt from
    its start), one where there is work for every slot; key runs for few, long tiles."""
    ops = _ops()

    def shape(seqs, nkv=8, group=4, window=0):
        ctx = SimpleNamespace(h_seq_starts=[a for a, _ in seqs], h_seq_lens=[n for _, n in seqs],
                              token_ids=torch.zeros(1, dtype=torch.int32, device=DEV), extra={})
        return ops._prefill_shape(ops.AttentionPlan(ctx, group, 128), nkv, window, 128)

    assert shape([(0, 2048)]) == (2, 1)
    assert shape([(0, 1024)]) == (2, 1)  # runs would cost more than they save: the tiles are short on average
    assert shape([(0, 8192)]) == (1, 1)
    assert shape([(0, 4096)]) == (1, 1)
    assert shape([(2048, 2048)]) == (1, 1)  # work for every slot; the longest tile ends alone and fast
    assert shape([(3584, 512)]) == (1, 4)
    assert shape([(0, 2048)] * 4) == (1, 1)
    assert shape([(0, 20)]) == (1, 1)  # one step: nothing to share


@pytest.mark.parametrize("case", ATTN_CASES[:7], ids=lambda c: f"h{c[0]}kv{c[1]}d{c[2]}p{c[3]}w{c[4]}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_attention_generic(case, dtype):
    """The FMA kernel that serves what the matrix-core kernels refuse, called by itself."""
    ops = _ops()
    nq, nkv, d, page, window, seqs = case
    q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, dtype, seed=3 + d, window=window)
    out = torch.full_like(q, float("nan"))
    ops.attention_generic(q, kc, vc, out, ctx.positions, ctx.token_slot, table, page, nq, nkv, d, window,
                          1.0 / math.sqrt(d), ctx.max_position)
    if dtype == torch.float32:
        torch.testing.assert_close(out.cpu(), want, rtol=1e-5, atol=2e-6)
    else:
        _close_bf16_attention(out.float().cpu(), want, seqs, "generic")


@pytest.mark.parametrize("d", [24, 40, 8, 200])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_attention_of_head_sizes_between_the_matrix_cores_steps(d, dtype):
    """Head sizes that are multiples of 8 and not of 16 reach the kernel that takes any size
    through the same entry, in both types."""
    ops = _ops()
    nq, nkv, page = 6, 2, 4
    seqs = [(9, 1), (0, 21), (150, 1), (40, 13)]
    q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, dtype, seed=d)
    out = torch.full_like(q, float("nan"))
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, 0, 1.0 / math.sqrt(d))
    if dtype == torch.float32:
        torch.testing.assert_close(out.cpu(), want, rtol=1e-5, atol=2e-6)
    else:
        _close_bf16_attention(out.float().cpu(), want, seqs, f"head size {d}")


def test_attention_f32_head_size_off_the_grid_takes_the_generic_kernel():
    ops = _ops()
    nq, nkv, d, page = 6, 2, 24, 4
    q, kc, vc, table, ctx, want = _paged_problem([(9, 1), (0, 21)], nq, nkv, d, page, torch.float32, seed=2)
    out = torch.full_like(q, float("nan"))
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, 0, 1.0 / math.sqrt(d))
    torch.testing.assert_close(out.cpu(), want, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("far", [3, 257, 640])
def test_attention_finds_a_far_key(dtype, far):
    """One key among hundreds holds the mass: a kernel that skips or misplaces its page
    returns something far from that key's value (7.0 in every channel)."""
    ops = _ops()
    nq, nkv, d, page = 8, 2, 128, 16
    for seqs, who in (([(699, 1), (10, 1)], 0), ([(5, 1), (100, 600)], 1)):
        q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, dtype, seed=far, spike=(who, far))
        out = torch.empty_like(q)
        ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, 0, 1.0 / math.sqrt(d))
        got = out.float().cpu()
        row = 0 if who == 0 else got.shape[0] - 1
        assert (want[row] > 6.5).all()  # the construction works in the plain attention
        torch.testing.assert_close(got[row], want[row], rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(got, want, rtol=2e-2, atol=2e-2)


def _decode_splits(ops, context, nkv, page):
    """(keys per split, splits) of a decode launch of one request of ``context`` keys: the host
    lays out splits of at most ``chunk`` keys, the kernel deals the request's keys to them evenly
    in runs of a multiple of 32, at least 128."""
    pairs = nkv
    want = max(1, ops.chip().units // pairs)
    chunk = max(ops._MIN_SPLIT_KEYS, -(-(-(-context // want)) // 128) * 128)
    chunk = min(chunk, max(32, ((ops._MAX_SPLIT_PAGES - 1) * page - 31) // 32 * 32))
    nsplit = -(-context // chunk)
    run = min(max((-(-context // nsplit) + 31) // 32 * 32, 128), chunk)
    return run, nsplit


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("context", [9000, 16000, 20000])
def test_decode_attention_finds_a_key_wherever_the_splits_fall(dtype, context):
    """A single token over thousands of keys, cut into many splits: the key that holds the mass
    is the first of a split, the last of the split before, the first and the last of the last
    split (the token's own), and the very first.  A split that is dropped, merged with a wrong
    weight or read one key short loses the value 7.0."""
    ops = _ops()
    nq, nkv, d, page = 8, 2, 128, 16
    chunk, nsplit = _decode_splits(ops, context, nkv, page)
    assert nsplit >= 30 and chunk % 128 == 0
    middle = (nsplit // 2) * chunk
    for far in (0, middle, middle - 1, (nsplit - 1) * chunk, context - 1):
        seqs = [(context - 1, 1)]
        q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, dtype, seed=context + far, spike=(0, far))
        out = torch.full_like(q, float("nan"))
        ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, 0, 1.0 / math.sqrt(d))
        got = out.float().cpu()
        assert (want[0] > 6.5).all()  # the construction works in the plain attention
        tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=0)
        torch.testing.assert_close(got, want, **tol)


@pytest.mark.parametrize("far", [0, 8191, 8192, 15999, 16000, 16149])
def test_prefill_attention_finds_a_key_behind_a_long_prefix(far):
    """150 tokens of a prompt behind 16,000 cached ones: few, long tiles whose keys are cut into
    runs and merged.  The last query's mass sits on a key at the prefix's start, at a run's edge,
    at the prefix's end, at the portion's first token and on the query's own."""
    ops = _ops()
    nq, nkv, d, page = 8, 2, 128, 16
    seqs = [(16000, 150)]
    q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, torch.bfloat16, seed=far + 1, spike=(0, far))
    out = torch.full_like(q, float("nan"))
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, 0, 1.0 / math.sqrt(d))
    got = out.float().cpu()
    assert (want[-1] > 6.5).all()
    torch.testing.assert_close(got[-1], want[-1], rtol=1e-2, atol=0)
    # the other rows hold the spike's value too where their own scores let it through: all rows
    _close_bf16_attention(got, want, seqs, f"long prefix, key {far}")


def test_attention_window_edge():
    """Keys exactly at and just outside the window's edge: the key one step too far holds a
    huge value; it must not leak into the result."""
    ops = _ops()
    nq, nkv, d, page, window = 4, 2, 64, 8, 33
    for dtype in (torch.float32, torch.bfloat16):
        for seqs in ([(100, 1)], [(60, 41)]):
            q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, dtype, seed=5, window=window)
            out = torch.empty_like(q)
            ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, window, 1.0 / math.sqrt(d))
            if dtype == torch.float32:
                torch.testing.assert_close(out.cpu(), want, rtol=1e-5, atol=2e-6)
            else:
                _close_bf16_attention(out.float().cpu(), want, seqs, "window edge")


@pytest.mark.parametrize("page", [16, 4], ids=["p16", "p4"])
def test_prefill_attention_reads_nothing_usable_behind_the_window(page):
    """Pages that lie wholly behind the window of a portion's first token have been given back:
    here they hold NaN, keys and values, and so does everything after the last token.  The
    tiles' first and last steps still touch them; nothing of it may reach a product."""
    ops = _ops()
    nq, nkv, d, window = 8, 2, 128, 100
    seqs = [(700, 150), (90, 40), (0, 260)]
    q, kc, vc, table, ctx, want = _paged_problem(seqs, nq, nkv, d, page, torch.bfloat16, seed=11, window=window)
    slot_of = {}
    for tok, slot in enumerate(ctx.token_slot.tolist()):
        slot_of.setdefault(slot, ctx.positions[tok].item())  # the portion's first position
    host_table = table.cpu()
    poisoned = 0
    for slot, first in slot_of.items():
        gone = max(0, first - window + 1) // page  # pages whose every key is out of every row's window
        for pid in host_table[slot, :gone].tolist():
            kc[pid] = float("nan")
            vc[pid] = float("nan")
            poisoned += 1
    assert poisoned > 10
    out = torch.full_like(q, float("nan"))
    ops.paged_attention(q, kc, vc, out, ctx, table, page, nq, nkv, d, window, 1.0 / math.sqrt(d))
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    _close_bf16_attention(got, want, seqs, "behind the window")


# --------------------------------------------------------------------------- #
# norms, activation, rotation, cache write, products, embedding, arg-max
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("hidden", [80, 333, 1000, 4096, 5120, 16384, 20000])
def test_add_rmsnorm(dtype, hidden):
    ops = _ops()
    t = 37
    res = torch.randn(t, hidden)
    delta = torch.randn(t, hidden).to(dtype)
    w = 1 + 0.1 * torch.randn(hidden)
    eps = 3e-5
    want_res = res + delta.float()
    want = plain_rmsnorm(want_res, w, eps)
    r = res.to(DEV)
    out = torch.empty(t, hidden, dtype=dtype, device=DEV)
    ops.add_rmsnorm(r, delta.to(DEV), w.to(DEV), out, eps)
    torch.testing.assert_close(r.cpu(), want_res, rtol=0, atol=0)  # residual updated in place
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=8e-3, atol=8e-3)
    torch.testing.assert_close(out.float().cpu(), want, **tol)
    # without a delta, and for chosen rows only
    rows = torch.tensor([5, 0, 36], dtype=torch.int32)
    out2 = torch.empty(3, hidden, dtype=dtype, device=DEV)
    ops.add_rmsnorm(r, None, w.to(DEV), out2, eps, rows.to(DEV))
    torch.testing.assert_close(out2.float().cpu(), want[rows.long()], **tol)
    # unit RMS with weight one
    ones = torch.ones(hidden, device=DEV)
    out3 = torch.empty(t, hidden, dtype=torch.float32, device=DEV)
    ops.add_rmsnorm(r, None, ones, out3, 0.0)
    torch.testing.assert_close(out3.square().mean(-1).cpu(), torch.ones(t), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_swiglu(dtype):
    ops = _ops()
    _swiglu_case(dtype, 19, 333)  # odd width: one element per thread
    _swiglu_case(dtype, 70, 12288)  # eight per thread


def _swiglu_case(dtype, t, inter):
    ops = _ops()
    x = torch.randn(t, 2 * inter).to(dtype)
    want = torch.nn.functional.silu(x[:, :inter].float()) * x[:, inter:].float()
    out = torch.empty(t, inter, dtype=dtype, device=DEV)
    ops.swiglu(x.to(DEV), out)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=8e-3, atol=8e-3)
    torch.testing.assert_close(out.float().cpu(), want, **tol)
    x[:, :inter] = 0  # zero gate => zero
    ops.swiglu(x.to(DEV), out)
    assert (out == 0).all()


def test_rope_table_matches_plain():
    ops = _ops()
    for d, theta in ((16, 1e4), (48, 5e5), (128, 1e6)):
        cos, sin = ops.rope_table(plain_inv_freq(d, theta).to(DEV), 5000)
        wc, ws = plain_rope_tables(torch.arange(5000), d, theta)
        torch.testing.assert_close(cos.cpu(), wc, rtol=0, atol=1e-7)
        torch.testing.assert_close(sin.cpu(), ws, rtol=0, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", [(5, 5, 48, 8), (6, 2, 128, 16), (3, 1, 16, 4), (4, 4, 256, 4)])
@pytest.mark.parametrize("many", [False, True], ids=["few", "many"])
def test_qknorm_rope_kvwrite(dtype, shape, many):
    ops = _ops()
    nq, nkv, d, page = shape
    theta, eps = 77777.0, 2e-5
    if many:  # enough tokens for the value tile kernel: runs that line up with pages and runs that do not
        positions = list(range(3, 40)) + list(range(96, 117)) + [7] + list(range(4000, 3990, -1))
        slots = [2] * 37 + [0] * 21 + [1] + [3] * 10
    else:
        positions = [0, 1, 2, 9, 300, 301, 4000]
        slots = [2, 2, 2, 0, 1, 1, 3]
    t = len(positions)
    qkv = torch.randn(t, (nq + 2 * nkv) * d).to(dtype)
    qw = 1 + 0.1 * torch.randn(d)
    kw = 1 + 0.1 * torch.randn(d)
    max_pages = 4001 // page + 1
    table = torch.zeros((4, max_pages), dtype=torch.int32)
    pid = 1
    for p, s in sorted(zip(positions, slots), key=lambda ps: (ps[0] * 7 + ps[1]) % 13):  # pages in no order
        if table[s, p // page] == 0:
            table[s, p // page] = pid
            pid += 1
    kc = torch.full((pid, nkv, page, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((pid, nkv, d, page), float("nan"), dtype=dtype, device=DEV)
    cos, sin = ops.rope_table(plain_inv_freq(d, theta).to(DEV), 4001)
    q_out = torch.empty(t, nq * d, dtype=dtype, device=DEV)
    ops.qknorm_rope_kvwrite(
        qkv.to(DEV), q_out, kc, vc, qw.to(DEV), kw.to(DEV), cos, sin,
        torch.tensor(positions, dtype=torch.int32, device=DEV),
        torch.tensor(slots, dtype=torch.int32, device=DEV), table.to(DEV), page, nq, nkv, d, eps, max(positions),
    )
    x = qkv.float()
    q = x[:, : nq * d].view(t, nq, d)
    k = x[:, nq * d : (nq + nkv) * d].view(t, nkv, d)
    v = x[:, (nq + nkv) * d :].view(t, nkv, d)
    pc, ps = plain_rope_tables(torch.tensor(positions), d, theta)
    want_q = plain_rope_apply(plain_rmsnorm(q, qw, eps), pc, ps).reshape(t, nq * d)
    want_k = plain_rope_apply(plain_rmsnorm(k, kw, eps), pc, ps)
    tol = dict(rtol=1e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=8e-3, atol=8e-3)
    torch.testing.assert_close(q_out.float().cpu(), want_q, **tol)
    kc, vc = kc.float().cpu(), vc.float().cpu()
    written_k = torch.zeros_like(kc, dtype=torch.bool)
    for i, (p, s) in enumerate(zip(positions, slots)):
        page_id, off = int(table[s, p // page]), p % page
        torch.testing.assert_close(kc[page_id, :, off, :], want_k[i], **tol)
        torch.testing.assert_close(vc[page_id, :, :, off], v[i], rtol=0, atol=0)
        written_k[page_id, :, off, :] = True
    assert torch.isnan(kc[~written_k]).all()  # nothing else was touched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("case", [
    # nq, nkv, d, page, channels that rotate, pairing
    (4, 2, 64, 8, 32, "half_split"),     # the first half of the head only
    (4, 2, 64, 8, 64, "interleaved"),    # pairs (2i, 2i + 1) over the whole head
    (6, 3, 48, 4, 16, "interleaved"),    # a third of the head, interleaved
    (3, 1, 128, 16, 64, "half_split"),
    (2, 2, 24, 4, 12, "half_split"),     # a head size that no vector access divides evenly
    (5, 5, 256, 8, 2, "interleaved"),    # one pair
], ids=lambda c: f"h{c[0]}kv{c[1]}d{c[2]}r{c[4]}{c[5]}")
@pytest.mark.parametrize("many", [False, True], ids=["few", "many"])
def test_qknorm_rope_in_other_pairings_and_widths(dtype, case, many):
    """How a rotation is applied is the position part's to say: the first ``rotary_dim`` channels
    of a head rotate, as half-split or as interleaved pairs, the rest pass with the norm alone.
    Against the rotation written as a complex product."""
    ops = _ops()
    nq, nkv, d, page, rot, pairing = case
    theta, eps = 5000.0, 1e-5
    positions = (list(range(2, 31)) + [90, 91, 400]) if many else [0, 1, 5, 400]
    slots = ([1] * 29 + [0, 0, 2]) if many else [1, 1, 0, 2]
    t = len(positions)
    gen = torch.Generator().manual_seed(d + rot)
    qkv = torch.randn((t, (nq + 2 * nkv) * d), generator=gen).to(dtype)
    qw = 1 + 0.1 * torch.randn(d, generator=gen)
    kw = 1 + 0.1 * torch.randn(d, generator=gen)
    table = torch.zeros((3, 401 // page + 1), dtype=torch.int32)
    pid = 1
    for p, s in zip(positions, slots):
        if table[s, p // page] == 0:
            table[s, p // page] = pid
            pid += 1
    kc = torch.full((pid, nkv, page, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((pid, nkv, d, page), float("nan"), dtype=dtype, device=DEV)
    inv = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float32) / rot))
    cos, sin = ops.rope_table(inv.to(DEV), 401)
    assert cos.shape == (401, rot // 2)
    q_out = torch.empty(t, nq * d, dtype=dtype, device=DEV)
    ops.qknorm_rope_kvwrite(
        qkv.to(DEV), q_out, kc, vc, qw.to(DEV), kw.to(DEV), cos, sin,
        torch.tensor(positions, dtype=torch.int32, device=DEV),
        torch.tensor(slots, dtype=torch.int32, device=DEV), table.to(DEV), page, nq, nkv, d, eps, max(positions),
        pairing,
    )
    x = qkv.float()
    q = x[:, : nq * d].view(t, nq, d)
    k = x[:, nq * d : (nq + nkv) * d].view(t, nkv, d)
    v = x[:, (nq + nkv) * d :].view(t, nkv, d)
    pos = torch.tensor(positions)
    want_q = rotate_pairs(plain_rmsnorm(q, qw, eps), pos, rot, theta, pairing).reshape(t, nq * d)
    want_k = rotate_pairs(plain_rmsnorm(k, kw, eps), pos, rot, theta, pairing)
    tol = dict(rtol=1e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=8e-3, atol=8e-3)
    torch.testing.assert_close(q_out.float().cpu(), want_q, **tol)
    # the channels beyond the rotated ones are the normed input, whatever the position
    if rot < d:
        torch.testing.assert_close(
            q_out.float().cpu().view(t, nq, d)[..., rot:], plain_rmsnorm(q, qw, eps)[..., rot:], **tol)
    kc, vc = kc.float().cpu(), vc.float().cpu()
    for i, (p, s) in enumerate(zip(positions, slots)):
        page_id, off = int(table[s, p // page]), p % page
        torch.testing.assert_close(kc[page_id, :, off, :], want_k[i], **tol)
        torch.testing.assert_close(vc[page_id, :, :, off], v[i], rtol=0, atol=0)
    with pytest.raises(ops.KernelError, match="pairing"):
        ops.qknorm_rope_kvwrite(
            qkv.to(DEV), q_out, kc.to(DEV, dtype), vc.to(DEV, dtype), qw.to(DEV), kw.to(DEV), cos, sin,
            torch.tensor(positions, dtype=torch.int32, device=DEV),
            torch.tensor(slots, dtype=torch.int32, device=DEV), table.to(DEV), page, nq, nkv, d, eps, max(positions),
            "by_threes",
        )


@pytest.mark.parametrize("shape", [(1, 96, 64), (7, 503, 96), (130, 200, 333), (64, 64, 16), (33, 48, 7),
                                   (40, 1000, 4100), (19, 70, 130)])
def test_gemm_f32(shape):
    ops = _ops()
    m, n, k = shape
    a, w = torch.randn(m, k), torch.randn(n, k)
    out = torch.empty(m, n, device=DEV)
    ops.gemm_f32(a.to(DEV), w.to(DEV), out)
    want = (a.double() @ w.double().T).float()
    torch.testing.assert_close(out.cpu(), want, rtol=1e-5, atol=1e-5 * math.sqrt(k))
    # a row's result does not depend on the rows beside it, nor on the tiling that their
    # number selects (1, up to 16, up to 32, more)
    for lo, hi in [(m // 2, m // 2 + 1), (0, min(m, 9)), (max(0, m - 20), m), (max(0, m - 33), m)]:
        part = torch.empty(hi - lo, n, device=DEV)
        ops.gemm_f32(a[lo:hi].to(DEV), w.to(DEV), part)
        assert torch.equal(part, out[lo:hi]), (shape, lo, hi)
    # views: rows of wider matrices, a start that is not 16-byte aligned
    wide_a = torch.randn(m, k + 5).to(DEV)
    wide_w = torch.randn(n, k + 5).to(DEV)
    wide_out = torch.zeros(m, n + 3, device=DEV)
    ops.gemm_f32(wide_a[:, 1 : k + 1], wide_w[:, 1 : k + 1], wide_out[:, 2 : n + 2])
    ref = (wide_a[:, 1 : k + 1].double() @ wide_w[:, 1 : k + 1].double().T).float()
    torch.testing.assert_close(wide_out[:, 2 : n + 2], ref, rtol=1e-5, atol=1e-5 * math.sqrt(k))
    assert float(wide_out[:, :2].abs().max()) == 0.0 and float(wide_out[:, n + 2 :].abs().max()) == 0.0


def test_gemm_f32_keeps_what_bfloat16_would_lose():
    """A true float32 product: a term 2^-12 of its neighbours survives (it would vanish in a
    product with bfloat16 or tf32-like operands)."""
    ops = _ops()
    k = 64
    a = torch.ones(1, k)
    w = torch.ones(1, k)
    w[0, 17] = 1.0 + 2.0 ** -12
    out = torch.empty(1, 1, device=DEV)
    ops.gemm_f32(a.to(DEV), w.to(DEV), out)
    assert out.item() == k + 2.0 ** -12


@pytest.mark.parametrize("shape", [(1, 503, 96), (8, 4096, 4096), (16, 300, 1000), (64, 1000, 12288), (17, 6144, 4096), (200, 331, 80), (3, 24, 48),
                                   (8, 6144, 4096), (1, 5000, 256), (16, 4618, 1160), (11, 6120, 96)])  # the last four: workgroups of 24 weight rows
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["bf16out", "f32out"])
def test_gemm_bf16(shape, out_dtype):
    ops = _ops()
    m, n, k = shape
    a = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    got = ops.gemm_bf16(a.to(DEV), w.to(DEV), out_dtype)
    want = a.float() @ w.float().T
    tol = dict(rtol=1e-2, atol=1e-2) if got.dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(got.float().cpu(), want, **tol)


@pytest.mark.parametrize("shape", [(1, 320, 96), (8, 12288, 4096), (16, 176, 80), (13, 100, 64), (5, 24, 200)])
def test_gemm_bf16_swiglu_fused(shape):
    ops = _ops()
    m, inter, k = shape
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(2 * inter, k) / math.sqrt(k)).bfloat16()
    got = ops.gemm_bf16_swiglu(x.to(DEV), w.to(DEV))
    gu = (x.float() @ w.float().T).bfloat16().float()
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    torch.testing.assert_close(got.float().cpu(), want, rtol=2e-2, atol=2e-2)
    if ops.rows_plan(33, inter, k, swiglu=True) is None and not ops._tile_applies(33, 2 * inter, k, inter):
        assert ops.gemm_bf16_swiglu(torch.zeros(33, k, dtype=torch.bfloat16, device=DEV), w.to(DEV)) is None


# rows, result columns, K: row counts around the blocks of 16 and 64 rows, column counts that end
# inside a workgroup's 64 (or 32) columns and inside a lane's four, one chunk of K and many
TILE_SHAPES = [(17, 2048, 128), (33, 2052, 384), (64, 4096, 1024), (96, 2116, 256), (130, 3000, 640),
               (256, 6144, 1024), (200, 2048, 3072), (300, 2048, 256), (512, 4096, 1024)]


@pytest.mark.parametrize("shape", TILE_SHAPES)
def test_tile_product_of_small_matrices(shape):
    """17 to 512 rows over a matrix of a few megabytes run one kernel of this package instead of
    the library's; against the float32 product of the same bfloat16 operands."""
    ops = _ops()
    m, n, k = shape
    assert ops._tile_applies(m, n, k, n)
    a = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    w[n - 1] = 3.0 / math.sqrt(k)  # the last weight row and the last row of x stand out:
    a[m - 1] = 1.0                 # a clamped or dropped edge shows
    got = ops.gemm_bf16(a.to(DEV), w.to(DEV), torch.bfloat16)
    assert got.dtype == torch.bfloat16 and got.shape == (m, n)
    want = a.float() @ w.float().T
    torch.testing.assert_close(got.float().cpu(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("shape", [(17, 1024, 128), (40, 1028, 384), (64, 3072, 1024), (100, 1500, 256), (256, 3072, 1024), (500, 1024, 384)])
def test_tile_product_with_swiglu(shape):
    """The same kernel on the packed gate and up matrices, the activation in its epilogue:
    silu(gate) * up of the products rounded to bfloat16, as the unfused path computes it."""
    ops = _ops()
    m, inter, k = shape
    assert ops._tile_applies(m, 2 * inter, k, inter)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(2 * inter, k) / math.sqrt(k)).bfloat16()
    w[inter - 1] = 2.0 / math.sqrt(k)      # the last gate row
    w[2 * inter - 1] = -2.0 / math.sqrt(k)  # and the last up row
    x[m - 1] = 1.0
    got = ops.gemm_bf16_swiglu(x.to(DEV), w.to(DEV))
    assert got is not None and got.shape == (m, inter)
    gu = (x.float() @ w.float().T).bfloat16().float()
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    torch.testing.assert_close(got.float().cpu(), want, rtol=2e-2, atol=2e-2)


def test_tile_product_keeps_to_its_sizes():
    """Few rows, many rows, large matrices, narrow ones and a K that is no multiple of 128 go
    where they went before (the few-row kernel, the library)."""
    ops = _ops()
    assert not ops._tile_applies(16, 4096, 1024, 4096)
    assert not ops._tile_applies(513, 4096, 1024, 4096)
    assert not ops._tile_applies(64, 4096, 2048, 4096)   # 16 MB: the library is as fast
    assert not ops._tile_applies(64, 1024, 2048, 1024)   # too few workgroups
    assert not ops._tile_applies(64, 4096, 1000, 4096)
    assert not ops._tile_applies(64, 4098, 1024, 4098)
    x = torch.randn(64, 1000).bfloat16()
    w = (torch.randn(4096, 1000) / 30).bfloat16()
    got = ops.gemm_bf16(x.to(DEV), w.to(DEV), torch.bfloat16)
    torch.testing.assert_close(got.float().cpu(), x.float() @ w.float().T, rtol=1e-2, atol=1e-2)


# rows, result columns, K: more (gate, up) pairs of tiles than the chip has compute units; pairs that
# do not divide among the workgroups; a K whose chunks do not divide among the waves
STREAM_SHAPES = [(8, 12288, 4096), (1, 11200, 1024), (16, 4112, 1152), (5, 25600, 1280), (13, 8192, 2048)]


@pytest.mark.parametrize("shape", STREAM_SHAPES)
@pytest.mark.parametrize("scaled", [False, True], ids=["plain", "scaled"])
def test_gate_up_product_that_streams_several_pairs_a_workgroup(shape, scaled):
    """The few-row gate/up product of a matrix with more pairs of tiles than compute units walks
    several pairs in one workgroup.  Against the float32 reference, and bit for bit against the
    kernel of one pair a workgroup (the same sums in the same order)."""
    import ctypes

    ops = _ops()
    core = ops.core()
    m, inter, k = shape
    gen = torch.Generator().manual_seed(inter + k)
    x = torch.randn((m, k), generator=gen).bfloat16()
    w = (torch.randn((2 * inter, k), generator=gen) / math.sqrt(k)).bfloat16()
    w[inter - 1] = 2.0 / math.sqrt(k)       # the last gate row
    w[2 * inter - 1] = -2.0 / math.sqrt(k)  # and the last up row stand out
    xd, wd = x.to(DEV), w.to(DEV)
    partial = None
    factor = torch.ones(m, 1)
    if scaled:
        parts = 7
        partial = torch.rand((parts, 16), generator=gen) * k / parts
        factor = torch.rsqrt(partial[:, :m].sum(0) / k + 1e-6).reshape(m, 1)
        partial = partial.to(DEV)
    def run(nt):
        out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
        rc = core.rl_gemm_skinny_swiglu(
            ctypes.c_void_p(xd.data_ptr()), ctypes.c_void_p(wd.data_ptr()), ctypes.c_void_p(out.data_ptr()),
            m, inter, k, k, k, inter, nt, ops.chip().units, ctypes.c_void_p(partial.data_ptr() if scaled else 0),
            7 if scaled else 0, k if scaled else 0, ctypes.c_float(1e-6), ops._stream())
        assert rc == 0
        return out
    streamed, single = run(2), run(-2)
    assert torch.equal(streamed, single)
    gu = ((x.float() @ w.float().T) * factor).bfloat16().float()
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    torch.testing.assert_close(streamed.float().cpu(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("shape", [(1, 96, 64), (8, 4096, 4096), (16, 304, 1000), (5, 4096, 12288), (3, 40, 48)])
def test_products_fold_the_norm_between_them(shape):
    """producer: residual += x W^T, rows * weight, pieces of the sums of squares; consumer:
    takes those rows and scales its own result.  Together they are the product, the residual
    add, the norm and the next product (and the fused activation) of the unfused path."""
    from rapid_llm_amd.parts.lazy import ScaledRows

    ops = _ops()
    m, hidden, k = shape
    torch.manual_seed(m + hidden)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(hidden, k) / math.sqrt(k)).bfloat16()
    residual = torch.randn(m, hidden)
    norm_w = 1 + 0.1 * torch.randn(hidden)
    eps = 3e-6
    res = residual.clone().to(DEV)
    rows, partial = ops.gemm_bf16_residual(x.to(DEV), w.to(DEV), res, norm_w.to(DEV))
    delta = (x.float() @ w.float().T).bfloat16().float()
    want_res = residual + delta
    # the product is rounded to bfloat16 before the add; sums in another order may round a
    # few results one step the other way
    torch.testing.assert_close(res.cpu() - residual, delta, rtol=2.0 ** -7, atol=1e-5)
    assert float((res.cpu() - want_res).abs().gt(1e-5).float().mean()) < 0.01
    torch.testing.assert_close(rows.float().cpu(), (res.cpu() * norm_w).bfloat16().float(), rtol=8e-3, atol=1e-6)
    ss = partial.sum(0).cpu()[:m]
    torch.testing.assert_close(ss, (res.cpu() ** 2).sum(-1), rtol=1e-5, atol=1e-5)
    assert partial.shape[1] == 16 and float(partial[:, m:].abs().max() if m < 16 else 0.0) == 0.0
    # the consumer: a plain product, and the packed gate/up product with its activation
    scaled = ScaledRows(rows, partial, hidden, eps)
    normed = plain_rmsnorm(res.cpu(), norm_w, eps)
    n2 = 208
    # the second width takes workgroups of 24 weight rows (a tile and a half), the last of them short
    w2 = (torch.randn(n2, hidden) / math.sqrt(hidden)).bfloat16()
    for out_dtype, tol in ((torch.bfloat16, 2e-2), (torch.float32, 1e-2)):
        got = ops.gemm_bf16(rows, w2.to(DEV), out_dtype, scaled=scaled)
        want = normed.bfloat16().float() @ w2.float().T
        torch.testing.assert_close(got.float().cpu(), want, rtol=tol, atol=tol)
    # a width that takes workgroups of 24 weight rows (a tile and a half), the last of them short:
    # against the kernel's own order of operations (the rows as the producer rounded them, the
    # factor applied to the result), which leaves only the order of the float32 sums
    wide = 4616
    assert ops._skinny_tiles(m, wide, plain=True) == 3
    w3 = (torch.randn(wide, hidden) / math.sqrt(hidden)).bfloat16()
    factor = torch.rsqrt(ss / hidden + eps).reshape(m, 1)
    want = (rows.float().cpu() @ w3.float().T) * factor
    got = ops.gemm_bf16(rows, w3.to(DEV), torch.float32, scaled=scaled)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-4)
    got = ops.gemm_bf16(rows, w3.to(DEV), torch.bfloat16, scaled=scaled)
    torch.testing.assert_close(got.float().cpu(), want, rtol=1e-2, atol=1e-2)
    wgu = (torch.randn(2 * n2, hidden) / math.sqrt(hidden)).bfloat16()
    act = ops.gemm_bf16_swiglu(rows, wgu.to(DEV), scaled=scaled)
    gu = (normed.bfloat16().float() @ wgu.float().T).bfloat16().float()
    want = torch.nn.functional.silu(gu[:, :n2]) * gu[:, n2:]
    torch.testing.assert_close(act.float().cpu(), want, rtol=3e-2, atol=3e-2)
    # run again: the same bits (fixed orders of summation)
    res2 = residual.clone().to(DEV)
    rows2, partial2 = ops.gemm_bf16_residual(x.to(DEV), w.to(DEV), res2, norm_w.to(DEV))
    assert torch.equal(rows2, rows) and torch.equal(partial2, partial) and torch.equal(res2, res)


@pytest.mark.parametrize("shape", [(17, 4096, 4096), (64, 4096, 12288), (33, 200, 256), (48, 1000, 1280), (20, 64, 128),
                                   (65, 200, 256), (100, 4096, 4096), (130, 1000, 1280), (192, 1024, 2048)])
def test_product_in_runs_of_k_and_the_norm_that_adds_them(shape):
    """17 to 192 rows (beyond 64 in blocks of 64 rows): the product of a narrow matrix as float32
    runs of K, and the norm kernel that adds the runs, against the library product followed by
    the ordinary norm."""
    ops = _ops()
    m, n, k = shape
    assert m <= ops.MID_MAX_ROWS
    gen = torch.Generator().manual_seed(m + n)
    x = (torch.randn((m, k), generator=gen)).bfloat16()
    x[m - 1] = 1.0  # the last row stands out: a block of rows that stops short shows
    w = (torch.randn((n, k), generator=gen) * 0.05).bfloat16()
    assert ops.mid_runs(n, k) >= 1
    parts = ops.gemm_bf16_parts(x.to(DEV), w.to(DEV))
    assert parts.shape[1:] == (m, n) and parts.shape[0] == ops.mid_runs(n, k)
    want = x.float() @ w.float().T
    torch.testing.assert_close(parts.sum(0).cpu(), want, rtol=2e-3, atol=2e-3 * float(want.abs().max()))
    # the norm that adds them
    res = torch.randn((m, n), generator=gen)
    norm_w = 1 + 0.1 * torch.randn(n, generator=gen)
    eps = 1e-5
    got_res = res.to(DEV).clone()
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    ops.add_rmsnorm_parts(got_res, parts, norm_w.to(DEV), out, eps)
    delta = parts.sum(0).bfloat16().float().cpu()
    want_res = res + delta
    torch.testing.assert_close(got_res.cpu(), want_res, rtol=0, atol=2.0 ** -7 * float(delta.abs().max()))
    want_out = want_res * torch.rsqrt(want_res.pow(2).mean(-1, keepdim=True) + eps) * norm_w
    torch.testing.assert_close(out.float().cpu(), want_out, rtol=2e-2, atol=2e-2)
    # the same twice: no order of summation is left to chance
    res2 = res.to(DEV).clone()
    out2 = torch.empty_like(out)
    ops.add_rmsnorm_parts(res2, ops.gemm_bf16_parts(x.to(DEV), w.to(DEV)), norm_w.to(DEV), out2, eps)
    assert torch.equal(res2, got_res) and torch.equal(out2, out)


# rows, result columns, K, SwiGLU, float32 result: every number of tiles a workgroup may hold
# (1, 2, 3, 6 tiles; 2, 3, 5 pairs), shares that leave some workgroups a tile short, more tiles
# than one round of workgroups holds (the vocabulary), 17 to 64 rows around the blocks of 16,
# one chunk of K (most waves then have none) and K that the waves do not share evenly
ROWS_SHAPES = [
    (17, 4096, 4096, False, False), (33, 6144, 2048, False, False), (48, 10240, 768, False, False),
    (64, 6144, 4096, False, False), (20, 16000, 512, False, False), (64, 19200, 384, False, True),
    (33, 151936, 256, False, True), (64, 151936, 128, False, True), (50, 2048, 4096, False, True),
    (17, 6144, 2048, True, False), (32, 12288, 4096, True, False), (64, 12288, 1152, True, False),
    (40, 17408, 256, True, False), (64, 17408, 256, True, False), (48, 20480, 384, True, False),
    (18, 3088, 1280, True, False),
]


@pytest.mark.parametrize("shape", ROWS_SHAPES, ids=lambda c: f"m{c[0]}n{c[1]}k{c[2]}{'sw' if c[3] else ''}{'f32' if c[4] else ''}")
def test_rows_product_of_wide_matrices(shape):
    """The product for 17 to 64 rows that keeps a chunk of X in registers for all the tiles a
    workgroup owns, through the entry points the parts call; the first and the last result
    columns, and those where one workgroup's share ends and the next begins, are checked like
    all others (every column's weights are its own)."""
    ops = _ops()
    m, n, k, swiglu, wide_out = shape
    gen = torch.Generator().manual_seed(m + n + k)
    x = torch.randn((m, k), generator=gen).bfloat16()
    w = (torch.randn(((2 if swiglu else 1) * n, k), generator=gen) / math.sqrt(k)).bfloat16()
    plan = ops.rows_plan(m, n, k, swiglu)
    assert plan is not None and not ops._tile_applies(m, w.shape[0], k, n)
    per, groups = plan
    assert ops.core().rl_gemm_rows_holds(int(swiglu), per, m) and -(-(n // 16) // groups) <= per
    before = ops.library_products
    if swiglu:
        got = ops.gemm_bf16_swiglu(x.to(DEV), w.to(DEV))
        gu = (x.float() @ w.float().T).bfloat16().float()
        want = torch.nn.functional.silu(gu[:, :n]) * gu[:, n:]
        tol = dict(rtol=2e-2, atol=2e-2)
    else:
        got = ops.gemm_bf16(x.to(DEV), w.to(DEV), torch.float32 if wide_out else torch.bfloat16)
        want = x.float() @ w.float().T
        tol = dict(rtol=1e-4, atol=1e-4) if wide_out else dict(rtol=1e-2, atol=1e-2)
    assert ops.library_products == before, "the product went to the library"
    assert got.shape == (m, n) and got.dtype == (torch.float32 if wide_out else torch.bfloat16)
    torch.testing.assert_close(got.float().cpu(), want, **tol)
    # the same bits every run: the waves' sums are added in a fixed order
    again = ops.gemm_bf16_swiglu(x.to(DEV), w.to(DEV)) if swiglu else ops.gemm_bf16(x.to(DEV), w.to(DEV), got.dtype)
    assert torch.equal(got, again)


def test_rows_product_refuses_what_it_was_not_built_for():
    import ctypes

    ops = _ops()
    core = ops.core()
    x = torch.zeros((64, 256), dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((2 * 25600, 256), dtype=torch.bfloat16, device=DEV)
    out = torch.zeros((64, 25600), dtype=torch.bfloat16, device=DEV)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    call = lambda m, n, k, sw, per, groups: core.rl_gemm_rows(P(x), P(w), P(out), m, n, k, k, k, n, sw, 1, per, groups, ops._stream())
    assert call(64, 25600, 256, 1, 5, 320) == 1   # five pairs beside 64 rows: not built
    assert call(48, 25600, 256, 1, 5, 320) == 0
    assert call(48, 25600, 256, 1, 5, 256) == 1   # a share of seven pairs in a workgroup that holds five
    assert call(48, 25600, 256, 1, 4, 400) == 1   # no kernel holds four pairs
    assert call(65, 25600, 256, 1, 5, 320) == 1 and call(48, 25608, 256, 1, 5, 321) == 1 and call(48, 25600, 200, 1, 5, 320) == 1
    torch.cuda.synchronize()
    assert ops.rows_plan(16, 12288, 4096, True) is None and ops.rows_plan(65, 12288, 4096, True) is None
    assert ops.rows_plan(33, 12288, 4000, True) is None and ops.rows_plan(33, 1000, 4096, False) is None
    assert ops.rows_plan(33, 1024, 4096, False) is None  # 64 tiles: too few workgroups to stream from
    assert ops.rows_plan(33, 25600, 5120, True) is None  # more than five pairs a compute unit: the library's


def test_wide_matrices_are_not_cut_into_runs_of_k():
    ops = _ops()
    assert ops.mid_runs(24576, 4096) == 0 and ops.mid_runs(151936, 4096) == 0
    assert ops.mid_runs(4096, 4096) == 4 and ops.mid_runs(4096, 12288) == 4
    assert ops.mid_runs(4096, 200) == 0  # K must be a multiple of 128
    assert ops.mid_runs(64, 128) == 1


def test_embed_takes_fed_tokens_from_the_sampling_buffer():
    """An id -(r + 1) reads row r of the buffer the sampling kernels write; other ids are
    the rows they name; an id that names no row of either reads row 0 and never faults."""
    ops = _ops()
    torch.manual_seed(9)
    table = torch.randn(37, 24)
    fed = torch.tensor([5, 36, 0, 11], dtype=torch.int32)
    ids = torch.tensor([3, -1, -4, 36, -2, -9, 99], dtype=torch.int32)
    out = torch.empty(len(ids), 24, dtype=torch.float32, device=DEV)
    ops.embed(ids.to(DEV), table.to(DEV), out, fed.to(DEV))
    want = table[[3, 5, 11, 36, 36, 0, 0]]
    assert torch.equal(out.cpu(), want)
    ops.embed(ids.to(DEV), table.to(DEV), out)  # no buffer: a negative id reads row 0
    assert torch.equal(out.cpu(), table[[3, 0, 0, 36, 0, 0, 0]])


def test_embed_and_argmax():
    ops = _ops()
    vocab, hidden = 503, 96
    for dtype in (torch.float32, torch.bfloat16):
        table = torch.randn(vocab, hidden).to(dtype)
        ids = torch.tensor([0, 502, 17, 17, 250], dtype=torch.int32)
        out = torch.empty(5, hidden, device=DEV)
        ops.embed(ids.to(DEV), table.to(DEV), out)
        assert torch.equal(out.cpu(), table.float()[ids.long()])
    logits = torch.randn(9, 151936)
    logits[3, 777] = logits[3, 90000] = 50.0  # a tie: the lower index wins
    out = torch.empty(9, dtype=torch.int32, device=DEV)
    ops.argmax(logits.to(DEV), out)
    assert out.cpu().tolist() == logits.argmax(-1).tolist()
    assert int(out[3]) == 777


PREPARED_CASES = [
    # nq, nkv, d, page, window, (tokens cached, tokens in the step) of every request
    (8, 2, 128, 16, 0, [(0, 70), (300, 1), (40, 33)]),     # portions beside a single token
    (6, 3, 64, 8, 0, [(100, 40), (5, 1), (0, 2)]),
    (4, 4, 192, 32, 57, [(400, 3), (20, 90)]),             # window
    (32, 8, 128, 16, 0, [(1000, 600)]),                    # few, long tiles: the keys cut into runs
]


@pytest.mark.parametrize("case", PREPARED_CASES, ids=lambda c: f"h{c[0]}kv{c[1]}d{c[2]}p{c[3]}w{c[4]}")
@pytest.mark.parametrize("normed", [True, False], ids=["norm", "nonorm"])
def test_attention_that_finishes_the_queries_itself(case, normed):
    """A step of portions and single tokens from the packed rows: the keys and values are
    normed, rotated and written by the head kernel (which leaves the queries alone), the
    attention kernels norm and rotate the query heads as they read them.  Against the plain
    formulas, and against the same step with the queries written out first."""
    ops = _ops()
    nq, nkv, d, page, window, seqs = case
    theta, eps = 50000.0, 3e-6
    gen = torch.Generator().manual_seed(d + nq + 1)
    rng = random.Random(nq * 17 + d)
    assert ops.attention_prepares_queries(torch.bfloat16, d, d // 2)
    total_pages = sum(-(-(a + n) // page) for a, n in seqs) + 1
    order = list(range(1, total_pages))
    rng.shuffle(order)
    max_pages = max(-(-(a + n) // page) for a, n in seqs) + 1
    table = torch.zeros((len(seqs) + 2, max_pages), dtype=torch.int32)
    kc = torch.full((total_pages, nkv, page, d), float("nan"))
    vc = torch.full((total_pages, nkv, d, page), float("nan"))
    slots = list(range(len(seqs) + 2))
    rng.shuffle(slots)
    qw = 1 + 0.1 * torch.randn(d, generator=gen) if normed else None
    kw = 1 + 0.1 * torch.randn(d, generator=gen) if normed else None
    rows, positions, token_slot, expect = [], [], [], []
    for i, (a, n) in enumerate(seqs):
        k_old = torch.randn(a, nkv, d, generator=gen).bfloat16().float()
        v_old = torch.randn(a, nkv, d, generator=gen).bfloat16().float()
        for p in range(-(-(a + n) // page)):
            pid = order.pop()
            table[slots[i], p] = pid
            lo, hi = p * page, min(a, (p + 1) * page)
            if hi > lo:
                kc[pid, :, : hi - lo, :] = k_old[lo:hi].transpose(0, 1)
                vc[pid, :, :, : hi - lo] = v_old[lo:hi].permute(1, 2, 0)
        raw = torch.randn(n, (nq + 2 * nkv) * d, generator=gen).bfloat16()
        rows.append(raw)
        q = raw.float()[:, : nq * d].view(n, nq, d)
        k = raw.float()[:, nq * d : (nq + nkv) * d].view(n, nkv, d)
        v = raw.float()[:, (nq + nkv) * d :].view(n, nkv, d)
        if normed:
            q, k = plain_rmsnorm(q, qw, eps), plain_rmsnorm(k, kw, eps)
        qpos = torch.arange(a, a + n)
        pc, ps = plain_rope_tables(qpos, d, theta)
        q, k = plain_rope_apply(q, pc, ps), plain_rope_apply(k, pc, ps)
        q, k = q.bfloat16().float(), k.bfloat16().float()  # what the products hold
        expect.append(
            plain_attention(q, torch.cat([k_old, k]), torch.cat([v_old, v]), d**-0.5, window or None, qpos,
                            torch.arange(a + n)).reshape(n, nq * d)
        )
        positions += list(range(a, a + n))
        token_slot += [slots[i]] * n
    tokens = len(positions)
    ctx = SimpleNamespace(
        positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
        token_slot=torch.tensor(token_slot, dtype=torch.int32, device=DEV),
        token_ids=torch.zeros(tokens, dtype=torch.int32, device=DEV),
        h_seq_starts=[a for a, _ in seqs], h_seq_lens=[n for _, n in seqs], max_position=max(positions), extra={},
    )
    cos, sin = ops.rope_table(plain_inv_freq(d, theta).to(DEV), max(positions) + 1)
    qkv = torch.cat(rows).to(DEV)
    tab = table.to(DEV)
    qwd, kwd = (qw.to(DEV), kw.to(DEV)) if normed else (None, None)
    want = torch.cat(expect)
    outs = []
    for in_kernel in (True, False):
        kcd, vcd = kc.bfloat16().to(DEV), vc.bfloat16().to(DEV)
        q_out = None if in_kernel else torch.full((tokens, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.qknorm_rope_kvwrite(qkv, q_out, kcd, vcd, qwd, kwd, cos, sin, ctx.positions, ctx.token_slot, tab, page,
                                nq, nkv, d, eps, ctx.max_position)
        out = torch.full((tokens, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.paged_attention(qkv if in_kernel else q_out, kcd, vcd, out, ctx, tab, page, nq, nkv, d, window, d**-0.5,
                            prepare=(qwd, cos, sin, eps) if in_kernel else None)
        got = out.float().cpu()
        assert torch.isfinite(got).all()
        _close_bf16_attention(got, want, seqs, "queries finished in the kernel" if in_kernel else "queries written out")
        outs.append(got)
    # the two ways round a query's channels alike but for the order of two multiplications
    assert (outs[0] - outs[1]).abs().max() <= 0.05 * want.abs().max()
    with pytest.raises(ops.KernelError, match="do not finish the queries"):
        ops.paged_attention(qkv.float(), kcd.float(), vcd.float(), out.float(), ctx, tab, page, nq, nkv, d, window,
                            d**-0.5, prepare=(qwd, cos, sin, eps))


FUSED_CASES = [
    # nq, nkv, d, page, window, cached lengths of the requests
    (8, 2, 128, 16, 0, [0, 5, 699, 31, 256]),
    (6, 3, 64, 4, 0, [17, 300, 1]),           # pages of four: values are read in two halves
    (20, 1, 64, 8, 0, [90, 513]),             # 20 heads on one kv head: two chunks of heads
    (4, 4, 192, 32, 57, [400, 20, 56, 57]),   # window
    (32, 8, 128, 16, 0, [2047] * 3),
]


@pytest.mark.parametrize("case", FUSED_CASES, ids=lambda c: f"h{c[0]}kv{c[1]}d{c[2]}p{c[3]}w{c[4]}")
@pytest.mark.parametrize("normed", [True, False], ids=["norm", "nonorm"])
def test_decode_attention_fused(case, normed):
    """Norm, rotation, cache write and split-key attention of a decode step in one
    kernel: the output and what lands in the cache against the plain formulas."""
    ops = _ops()
    nq, nkv, d, page, window, cached = case
    theta, eps = 50000.0, 3e-6
    gen = torch.Generator().manual_seed(d + nq)
    rng = random.Random(nq * 31 + d)
    n = len(cached)
    total_pages = sum(-(-(a + 1) // page) for a in cached) + 1
    order = list(range(1, total_pages))
    rng.shuffle(order)
    max_pages = max(-(-(a + 1) // page) for a in cached) + 1
    table = torch.zeros((n + 2, max_pages), dtype=torch.int32)
    kc = torch.full((total_pages, nkv, page, d), float("nan"))
    vc = torch.full((total_pages, nkv, d, page), float("nan"))
    slots = list(range(n + 2))
    rng.shuffle(slots)
    qw = 1 + 0.1 * torch.randn(d, generator=gen) if normed else None
    kw = 1 + 0.1 * torch.randn(d, generator=gen) if normed else None
    qkv = torch.randn(n, (nq + 2 * nkv) * d, generator=gen).bfloat16()
    expect, new_k, new_v = [], [], []
    for i, a in enumerate(cached):
        k_old = torch.randn(a, nkv, d, generator=gen).bfloat16().float()
        v_old = torch.randn(a, nkv, d, generator=gen).bfloat16().float()
        slot = slots[i]
        for p in range(-(-(a + 1) // page)):
            pid = order.pop()
            table[slot, p] = pid
            lo, hi = p * page, min(a, (p + 1) * page)
            if hi > lo:
                kc[pid, :, : hi - lo, :] = k_old[lo:hi].transpose(0, 1)
                vc[pid, :, :, : hi - lo] = v_old[lo:hi].permute(1, 2, 0)
        row = qkv[i].float()
        q = row[: nq * d].view(1, nq, d)
        k = row[nq * d : (nq + nkv) * d].view(1, nkv, d)
        v = row[(nq + nkv) * d :].view(1, nkv, d)
        if normed:
            q, k = plain_rmsnorm(q, qw, eps), plain_rmsnorm(k, kw, eps)
        pc, ps = plain_rope_tables(torch.tensor([a]), d, theta)
        q, k = plain_rope_apply(q, pc, ps), plain_rope_apply(k, pc, ps)
        k, q = k.bfloat16().float(), q.bfloat16().float()  # what the cache and the product hold
        keys, vals = torch.cat([k_old, k]), torch.cat([v_old, v])
        expect.append(
            plain_attention(q, keys, vals, d**-0.5, window or None, torch.tensor([a]), torch.arange(a + 1)).reshape(1, nq * d)
        )
        new_k.append(k[0])
        new_v.append(v[0])
    ctx = SimpleNamespace(
        positions=torch.tensor(cached, dtype=torch.int32, device=DEV),
        token_slot=torch.tensor(slots[:n], dtype=torch.int32, device=DEV),
        token_ids=torch.zeros(n, dtype=torch.int32, device=DEV),
        h_seq_starts=list(cached), h_seq_lens=[1] * n, max_position=max(cached), extra={},
    )
    assert ops.decode_attention_fusable(ctx, torch.bfloat16, nq // nkv, d, d // 2)
    cos, sin = ops.rope_table(plain_inv_freq(d, theta).to(DEV), max(cached) + 1)
    kcd, vcd = kc.bfloat16().to(DEV), vc.bfloat16().to(DEV)
    out = torch.full((n, nq * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    for _ in range(2):  # twice: the second launch finds the key it wrote itself
        ops.decode_attention_fused(
            qkv.to(DEV), kcd, vcd, out, ctx, table.to(DEV), page, nq, nkv, d, window, d**-0.5,
            qw.to(DEV) if normed else None, kw.to(DEV) if normed else None, cos, sin, eps, True,
        )
        got = out.float().cpu()
        assert torch.isfinite(got).all()
        _close_bf16_attention(got, torch.cat(expect), [(a, 1) for a in cached], "fused decode")
    kcc, vcc = kcd.float().cpu(), vcd.float().cpu()
    for i, a in enumerate(cached):
        pid, off = int(table[slots[i], a // page]), a % page
        torch.testing.assert_close(kcc[pid, :, off, :], new_k[i], rtol=8e-3, atol=8e-3)
        torch.testing.assert_close(vcc[pid, :, :, off], new_v[i], rtol=0, atol=0)
    # nothing else in the cache was touched
    before = kc.bfloat16().float()
    same = torch.isnan(before) == torch.isnan(kcc)
    for i, a in enumerate(cached):
        same[int(table[slots[i], a // page]), :, a % page, :] = True
    assert same.all()
