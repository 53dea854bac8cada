"""What fixes the plain implementation beside the reference's text: vectors the reference's
own tests hold, special cases that reduce to a library routine, and invariants; each chosen
so that a plausible mistake fails it (CPU only)."""

import math

import pytest
import torch
import torch.nn.functional as F

from plain_model import (
    plain_attention,
    plain_block,
    plain_forward,
    plain_greedy,
    plain_inv_freq,
    plain_layer_windows,
    plain_load,
    plain_rmsnorm,
    plain_rope_apply,
    plain_rope_tables,
    plain_swiglu_mlp,
)
from plain_sampler import plain_nucleus, plain_repetition_penalty, plain_sample
from tiny_configs import TINY, make_model_dir, random_tokens


# ---- RMSNorm ------------------------------------------------------------------------------
def test_rmsnorm_is_the_library_routine():
    x = torch.randn(7, 3, 48, dtype=torch.float64)
    w = 1 + 0.1 * torch.randn(48, dtype=torch.float64)
    torch.testing.assert_close(plain_rmsnorm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5))


def test_rmsnorm_unit_rms_and_eps_inside_the_root():
    x = torch.randn(5, 64) * 3
    y = plain_rmsnorm(x, torch.ones(64), 0.0)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(5))  # test_norm_activation.py:85
    # eps is added to the mean square, not to the root: a tiny input shows which
    tiny = torch.full((1, 4), 1e-4)
    assert abs(float(plain_rmsnorm(tiny, torch.ones(4), 1e-6)[0, 0]) - 1e-4 / math.sqrt(1e-8 + 1e-6)) < 1e-9


# ---- rotation -----------------------------------------------------------------------------
def test_inv_freq_vector():
    torch.testing.assert_close(plain_inv_freq(8, 10000.0), torch.tensor([1.0, 0.1, 0.01, 0.001]))


def test_rope_is_a_complex_multiplication_on_half_split_pairs():
    d, t = 16, 9
    x = torch.randn(t, 3, d, dtype=torch.float64)
    pos = torch.arange(5, 5 + t)
    cos, sin = plain_rope_tables(pos, d, 10000.0, torch.float64)
    got = plain_rope_apply(x, cos, sin)
    ang = torch.outer(pos.double(), plain_inv_freq(d, 10000.0).double())
    z = torch.complex(x[..., : d // 2], x[..., d // 2 :]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    torch.testing.assert_close(got, torch.cat((z.real, z.imag), dim=-1), atol=1e-6, rtol=1e-6)
    # pairing channel i with i + d/2, not 2i with 2i+1: the interleaved form differs
    inter = torch.view_as_real(torch.view_as_complex(x.reshape(t, 3, d // 2, 2).contiguous())
                               * torch.polar(torch.ones_like(ang), ang)[:, None, :]).reshape(t, 3, d)
    assert not torch.allclose(got, inter, atol=1e-3)


def test_rope_position_zero_is_identity_and_pairs_keep_their_norm():
    d = 32
    x = torch.randn(4, 2, d)
    cos, sin = plain_rope_tables(torch.zeros(4, dtype=torch.long), d, 1e6)
    torch.testing.assert_close(plain_rope_apply(x, cos, sin), x)  # test_rope_emb.py:57-125
    cos, sin = plain_rope_tables(torch.tensor([3, 50, 700, 9000]), d, 1e6)
    y = plain_rope_apply(x, cos, sin)
    torch.testing.assert_close(x[..., :16] ** 2 + x[..., 16:] ** 2, y[..., :16] ** 2 + y[..., 16:] ** 2,
                               atol=1e-5, rtol=1e-5)
    assert not torch.allclose(y[1], y[2])


def test_rope_scores_depend_on_distance_only_and_sign_is_counter_clockwise():
    d = 16
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)

    def score(pq, pk):
        cq, sq = plain_rope_tables(torch.tensor([pq]), d, 10000.0, torch.float64)
        ck, sk = plain_rope_tables(torch.tensor([pk]), d, 10000.0, torch.float64)
        return float((plain_rope_apply(q, cq, sq) * plain_rope_apply(k, ck, sk)).sum())

    assert abs(score(7, 3) - score(107, 103)) < 1e-6
    assert abs(score(7, 3) - score(3, 7)) > 1e-6
    # first pair, position 1, angle 1 rad: (1, 0) -> (cos 1, sin 1)
    e = torch.zeros(1, 1, d, dtype=torch.float64)
    e[0, 0, 0] = 1.0
    c, s = plain_rope_tables(torch.tensor([1]), d, 10000.0, torch.float64)
    r = plain_rope_apply(e, c, s)
    assert abs(float(r[0, 0, 0]) - math.cos(1.0)) < 1e-7 and abs(float(r[0, 0, d // 2]) - math.sin(1.0)) < 1e-7


# ---- attention ----------------------------------------------------------------------------
def test_attention_is_library_sdpa_with_repeat_interleave():
    t, nq, nkv, d = 11, 6, 2, 16
    q, k, v = torch.randn(t, nq, d), torch.randn(t, nkv, d), torch.randn(t, nkv, d)
    got = plain_attention(q, k, v, d**-0.5)
    g = nq // nkv
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(g, 0)[None],
        v.transpose(0, 1).repeat_interleave(g, 0)[None], is_causal=True, scale=d**-0.5,
    )[0].transpose(0, 1)
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    tiled = F.scaled_dot_product_attention(  # the wrong mapping, heads tiled (tests/reference.py:19-32)
        q.transpose(0, 1)[None], k.transpose(0, 1).repeat(g, 1, 1)[None],
        v.transpose(0, 1).repeat(g, 1, 1)[None], is_causal=True, scale=d**-0.5,
    )[0].transpose(0, 1)
    assert not torch.allclose(got, tiled, atol=1e-3)


def test_attention_one_head_last_row_is_plain_softmax():
    t, d = 6, 8
    q, k, v = torch.randn(t, 1, d), torch.randn(t, 1, d), torch.randn(t, 1, d)
    got = plain_attention(q, k, v, 0.5)
    want = torch.softmax((q[-1, 0] @ k[:, 0].T) * 0.5, -1) @ v[:, 0]
    torch.testing.assert_close(got[-1, 0], want)
    torch.testing.assert_close(got[0, 0], v[0, 0])  # the first token sees only itself


def test_attention_uniform_values_and_prefix_mask():
    t, d = 9, 8
    q, k = torch.randn(4, 2, d), torch.randn(t, 2, d)
    v = torch.full((t, 2, d), 3.5)
    out = plain_attention(q, k, v, 1.0, None, torch.arange(5, 9), torch.arange(t))
    torch.testing.assert_close(out, torch.full_like(out, 3.5))
    # with a prefix, query at position p sees keys <= p (rapid_llm/kernels/backend/cpu.py:89-101)
    v = torch.randn(t, 2, d)
    full = plain_attention(torch.randn(t, 2, d), k, v, 1.0)
    qq = torch.randn(t, 2, d)
    full = plain_attention(qq, k, v, 1.0)
    part = plain_attention(qq[5:], k, v, 1.0, None, torch.arange(5, 9), torch.arange(t))
    torch.testing.assert_close(part, full[5:])


def test_attention_window_counts_the_query_itself():
    t, d = 10, 8
    q, k, v = torch.randn(t, 1, d), torch.randn(t, 1, d), torch.randn(t, 1, d)
    one = plain_attention(q, k, v, 1.0, window=1)
    torch.testing.assert_close(one, v)  # a window of one position is the token itself
    three = plain_attention(q, k, v, 1.0, window=3)
    want = torch.softmax(q[7, 0] @ k[5:8, 0].T, -1) @ v[5:8, 0]
    torch.testing.assert_close(three[7, 0], want)


# ---- feed-forward -------------------------------------------------------------------------
def test_swiglu_is_silu_gate_times_up():
    x = torch.randn(5, 12)
    wg, wu, wd = torch.randn(20, 12), torch.randn(20, 12), torch.randn(12, 20)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    torch.testing.assert_close(plain_swiglu_mlp(x, wg, wu, wd), want)
    assert float(plain_swiglu_mlp(x, torch.zeros(20, 12), wu, wd).abs().max()) == 0.0  # zero gate
    assert not torch.allclose(plain_swiglu_mlp(x, wu, wg, wd), want)  # gate and up are not symmetric


# ---- the whole model ------------------------------------------------------------------------
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("plain")
    return {w: plain_load(make_model_dir(root, w, "float32"), torch.float64) for w in TINY}


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_only_distances_count(models, which):
    """Shifting every position leaves the logits alone.  A q/k norm applied after the rotation
    instead of before, with weights that differ by channel, would break this."""
    cfg, w = models[which]
    toks = random_tokens(40, cfg["vocab_size"], 1)
    # the angles are float32 products (rotary_embedding.py:194-202), hence 1e-6 and not 1e-12
    torch.testing.assert_close(plain_forward(cfg, w, toks), plain_forward(cfg, w, toks, position_offset=57),
                               atol=2e-6, rtol=0)


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_causal_and_prefix_consistent(models, which):
    cfg, w = models[which]
    toks = random_tokens(50, cfg["vocab_size"], 2)
    full = plain_forward(cfg, w, toks)
    torch.testing.assert_close(plain_forward(cfg, w, toks[:23]), full[:23], atol=1e-10, rtol=1e-10)
    other = list(toks)
    other[30] = (other[30] + 1) % cfg["vocab_size"]
    changed = plain_forward(cfg, w, other)
    torch.testing.assert_close(changed[:30], full[:30], atol=1e-10, rtol=1e-10)
    assert not torch.allclose(changed[30:], full[30:])


def _library_block(h, cfg, w, layer, order="reference"):
    """One block written a second time, from library routines alone (``F.rms_norm``,
    ``torch.polar``, ``F.scaled_dot_product_attention``, ``F.silu``, ``F.linear``), in the order
    of rapid_llm/models/base.py:231-266 (norm, mixer, add, norm, feed-forward, add) and :121-165
    (projection, head norms *before* the rotation, attention, output projection).  ``order``
    names a plausible misreading instead: the head norms after the rotation, or the norms
    behind the sub-layers (post-norm)."""
    p = f"model.layers.{layer}."
    eps, nq = cfg["rms_norm_eps"], cfg["num_attention_heads"]
    nkv, d, t = cfg["num_key_value_heads"], cfg["head_dim"], h.shape[0]
    angle = torch.outer(torch.arange(t, dtype=torch.float32), plain_inv_freq(d, cfg["rope_theta"])).double()
    unit = torch.polar(torch.ones_like(angle), angle)[:, None, :]

    def rotate(x):
        z = torch.complex(x[..., : d // 2], x[..., d // 2 :]) * unit
        return torch.cat((z.real, z.imag), dim=-1)

    def head_norm(x, name):
        return F.rms_norm(x, (d,), w[p + name], eps)

    def mixer(x):
        q = F.linear(x, w[p + "self_attn.q_proj.weight"]).view(t, nq, d)
        k = F.linear(x, w[p + "self_attn.k_proj.weight"]).view(t, nkv, d)
        v = F.linear(x, w[p + "self_attn.v_proj.weight"]).view(t, nkv, d)
        if order == "norm after rotation":
            q, k = head_norm(rotate(q), "self_attn.q_norm.weight"), head_norm(rotate(k), "self_attn.k_norm.weight")
        else:
            q, k = rotate(head_norm(q, "self_attn.q_norm.weight")), rotate(head_norm(k, "self_attn.k_norm.weight"))
        group = nq // nkv
        o = F.scaled_dot_product_attention(
            q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(group, 0)[None],
            v.transpose(0, 1).repeat_interleave(group, 0)[None], is_causal=True, scale=d**-0.5,
        )[0].transpose(0, 1).reshape(t, nq * d)
        return F.linear(o, w[p + "self_attn.o_proj.weight"])

    def feed_forward(x):
        gate, up = F.linear(x, w[p + "mlp.gate_proj.weight"]), F.linear(x, w[p + "mlp.up_proj.weight"])
        return F.linear(F.silu(gate) * up, w[p + "mlp.down_proj.weight"])

    n1 = lambda x: F.rms_norm(x, (x.shape[-1],), w[p + "input_layernorm.weight"], eps)
    n2 = lambda x: F.rms_norm(x, (x.shape[-1],), w[p + "post_attention_layernorm.weight"], eps)
    if order == "post-norm":
        h = n1(h + mixer(h))
        return n2(h + feed_forward(h))
    h = h + mixer(n1(h))
    return h + feed_forward(n2(h))


@pytest.mark.parametrize("which", ["A", "B", "E"])
def test_block_is_library_routines_in_the_references_order(models, which):
    """The order of a block (which norm feeds what, where the residual is added, the head norms
    before the rotation) is pinned by a second writing of the block from library routines; the
    two misreadings that a reader could fall into are shown to give other numbers, so the
    comparison could fail."""
    cfg, w = models[which]
    assert plain_layer_windows(cfg) == [None] * cfg["num_hidden_layers"]
    t = 23
    h = torch.randn(t, cfg["hidden_size"], dtype=torch.float64, generator=torch.Generator().manual_seed(8))
    for layer in range(cfg["num_hidden_layers"]):
        got = plain_block(h, cfg, w, layer, torch.arange(t), None)
        torch.testing.assert_close(got, _library_block(h, cfg, w, layer), atol=1e-9, rtol=1e-9)
        for wrong in ("norm after rotation", "post-norm"):
            other = _library_block(h, cfg, w, layer, wrong)
            # far beyond the comparison's tolerance (the sub-layers of a random model add little
            # to a stream of unit size, hence no larger a figure)
            assert float((other - got).abs().max()) > 1e-4, wrong
        h = got


def test_tied_and_untied_output(models):
    cfg, w = models["A"]
    assert cfg["tie_word_embeddings"] and "lm_head.weight" not in w
    toks = random_tokens(5, cfg["vocab_size"], 3)
    h = w["model.embed_tokens.weight"][torch.tensor(toks)]
    for layer in range(cfg["num_hidden_layers"]):
        h = plain_block(h, cfg, w, layer, torch.arange(5), None)
    h = plain_rmsnorm(h, w["model.norm.weight"], cfg["rms_norm_eps"])
    torch.testing.assert_close(plain_forward(cfg, w, toks), h @ w["model.embed_tokens.weight"].T)
    cfg_b, w_b = models["B"]
    assert "lm_head.weight" in w_b
    broken = {k: v for k, v in w_b.items() if k != "lm_head.weight"}
    with pytest.raises(KeyError):
        plain_forward(cfg_b, broken, [1, 2])


def test_window_layers_differ_from_full_ones(models):
    cfg, w = models["C"]
    assert plain_layer_windows(cfg) == [None, 21, 21]
    toks = random_tokens(60, cfg["vocab_size"], 4)
    windowed = plain_forward(cfg, w, toks)
    full = plain_forward({k: v for k, v in cfg.items() if k not in ("layer_types", "sliding_window")}, w, toks)
    torch.testing.assert_close(windowed[:21], full[:21], atol=1e-10, rtol=1e-10)  # inside the window
    assert not torch.allclose(windowed[30:], full[30:], atol=1e-6)


def test_greedy_continuation_feeds_back_its_own_tokens(models):
    cfg, w = models["A"]
    out = plain_greedy(cfg, w, [5, 9, 2], 4)
    assert out[0] == int(plain_forward(cfg, w, [5, 9, 2])[-1].argmax())
    assert out[1] == int(plain_forward(cfg, w, [5, 9, 2, out[0]])[-1].argmax())


# ---- sampling -------------------------------------------------------------------------------
def test_sampler_vectors_of_the_reference():
    # tests/engine/test_sampler.py:61-63, :229-266
    assert [plain_sample(torch.tensor(r), 0.0, 0.9, 0.5) for r in ([0.1, 0.9, 0.0], [0.5, 0.1, 0.4])] == [1, 0]
    torch.testing.assert_close(plain_repetition_penalty(torch.tensor([4.0, -4.0, 1.0]), [0, 1], 2.0),
                               torch.tensor([2.0, -8.0, 1.0]))
    torch.testing.assert_close(plain_repetition_penalty(torch.tensor([4.0, 0.0]), [0, 0, 0], 2.0),
                               torch.tensor([2.0, 0.0]))  # each token once
    torch.testing.assert_close(plain_repetition_penalty(torch.tensor([1.0, -2.0, 3.0]), [0, 2], 1.0),
                               torch.tensor([1.0, -2.0, 3.0]))
    # :66-72: top_p 0.1 keeps only the dominant token
    ids, kept = plain_nucleus(torch.tensor([0.7, 0.2, 0.1]), 0.1)
    assert ids.tolist() == [0, 1, 2] and kept.tolist() == [pytest.approx(0.7), 0.0, 0.0]
    for u in (0.0, 0.3, 0.999):
        assert plain_sample(torch.log(torch.tensor([0.7, 0.2, 0.1])), 1.0, 0.1, u) == 0


def test_nucleus_pool_and_flat_rows():
    probs = torch.softmax(torch.randn(500) * 3, 0)
    ids, kept = plain_nucleus(probs, 0.99, pool=16)
    assert set(ids.tolist()) == set(probs.topk(16).indices.tolist())  # :97-105: never beyond the pool
    flat = torch.full((2000,), 1 / 2000)
    ids, kept = plain_nucleus(flat, 0.999, pool=16)
    assert (kept > 0).all() and len(ids) == 16  # :108-121: a pool that never reaches top_p is kept whole
    # mass before a token decides: [0.5, 0.3, 0.2] with top_p 0.5 keeps two (0.5 is not > 0.5)
    _, kept = plain_nucleus(torch.tensor([0.5, 0.3, 0.2]), 0.5)
    assert (kept > 0).tolist() == [True, False, False] or (kept > 0).tolist() == [True, True, False]
    _, kept = plain_nucleus(torch.tensor([0.5, 0.3, 0.2]), 0.6)
    assert (kept > 0).tolist() == [True, True, False]


def test_draw_follows_the_distribution():
    logits = torch.log(torch.tensor([0.1, 0.6, 0.3]))
    picks = [plain_sample(logits, 1.0, 1.0, (i + 0.5) / 1000) for i in range(1000)]
    assert [picks.count(t) for t in range(3)] == [100, 600, 300]
    hot = [plain_sample(logits, 0.5, 1.0, (i + 0.5) / 1000) for i in range(1000)]
    assert hot.count(1) > 700  # a lower temperature sharpens
