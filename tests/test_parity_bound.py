"""The bfloat16 parity bound can fail (CPU only).

What the GPU tests compare an engine's logits with is the plain implementation; here the
"engine" is the plain implementation with a fault built in, and the same comparison has to
raise.  A plain result whose activations were rounded to bfloat16 wherever an engine rounds them
has to pass it.  No kernel is involved."""

import copy

import pytest
import torch

import parity
from plain_model import plain_forward, plain_load
from tiny_configs import TINY, make_model_dir, random_tokens


def _model(tmp_path, which):
    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, "bfloat16")
    pcfg, pw = plain_load(model_dir)
    return pcfg, pw, page, seed


def _rejects(got, want, label):
    with pytest.raises(AssertionError, match="bfloat16 logits are off"):
        parity.assert_bf16_close(got, want, label)


@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E", "F", "G", "H"])
def test_rounding_alone_passes_and_a_lost_key_does_not(tmp_path, which):
    pcfg, pw, page, seed = _model(tmp_path, which)
    n = min(pcfg["max_position_embeddings"], 200)
    toks = random_tokens(n, pcfg["vocab_size"], seed)
    want = plain_forward(pcfg, pw, toks)
    # rounding as an engine rounds: well inside the bound
    parity.assert_bf16_close(plain_forward(pcfg, pw, toks, cast=parity.to_bf16), want, f"{which}/rounded plain")
    # a key that every later query has lost (a page that was never written, a wrong slot)
    for key in (0, n // 4, n // 2, (n // 2 // page) * page):
        lost = plain_forward(pcfg, pw, toks, hide=lambda layer, q, k, key=key: (k[None, :] == key) & (q[:, None] > key))
        _rejects(lost, want, f"{which}/key {key} lost")
    # every query misses its own key (a step that reads the cache before it writes it)
    stale = plain_forward(pcfg, pw, toks, hide=lambda layer, q, k: (k[None, :] == q[:, None]) & (q[:, None] > 0))
    _rejects(stale, want, f"{which}/own key lost")
    # the same in one layer only, and only for the last 32 tokens (those decoded one by one)
    tail = plain_forward(
        pcfg, pw, toks,
        hide=lambda layer, q, k: (k[None, :] == q[:, None]) & (q[:, None] >= n - 32) & (layer == pcfg["num_hidden_layers"] - 1),
    )
    _rejects(tail, want, f"{which}/own key lost in the last layer's decoded tail")


def test_a_lost_run_of_keys_in_a_long_context(tmp_path):
    """One row at the end of 600 tokens: a run of 128 keys (one split of the decode kernel) is
    missed in one layer."""
    pcfg, pw, page, seed = _model(tmp_path, "D")
    n = 600
    toks = random_tokens(n, pcfg["vocab_size"], seed)
    want = plain_forward(pcfg, pw, toks)
    for lo in (0, 256, 384):
        lost = plain_forward(
            pcfg, pw, toks,
            hide=lambda layer, q, k, lo=lo: (k[None, :] >= lo) & (k[None, :] < lo + 128) & (q[:, None] == n - 1) & (layer == 0),
        )
        _rejects(lost[-1:], want[-1:], f"D/keys {lo}..{lo + 127} lost at the last row")


@pytest.mark.parametrize("which", ["C", "G"])
def test_a_window_off_by_one(tmp_path, which):
    pcfg, pw, page, seed = _model(tmp_path, which)
    n = 150
    toks = random_tokens(n, pcfg["vocab_size"], seed)
    want = plain_forward(pcfg, pw, toks)
    for delta in (-1, 1):
        other = copy.deepcopy(pcfg)
        other["sliding_window"] = pcfg["sliding_window"] + delta
        _rejects(plain_forward(other, pw, toks), want, f"{which}/window {delta:+d}")


def test_one_wrong_logit(tmp_path):
    pcfg, pw, page, seed = _model(tmp_path, "B")
    toks = random_tokens(40, pcfg["vocab_size"], seed)
    want = plain_forward(pcfg, pw, toks)
    got = want.clone()
    got[17, 300] += 0.1 * float(want.std())
    _rejects(got, want, "B/one logit moved by a tenth of the spread")
    assert parity.errors(got, want)[0] < parity.BF16_ROW  # the row figure alone would have missed it
