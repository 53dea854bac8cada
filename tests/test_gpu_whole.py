"""Each request alone and whole, float32 and bfloat16, against the plain implementation."""

import pytest
import torch

import parity
from plain_model import plain_forward, plain_load
from tiny_configs import TINY, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

F32_TOL = dict(rtol=2e-5, atol=3e-6)  # bfloat16: bounds relative to the logits' spread, see parity.py


def _runner(model_dir, dtype, page, **kw):
    from rapid_llm_amd import EngineConfig, ModelRunner

    body = dict(max_seq_len=kw.pop("max_seq_len", 128), page_size=page, num_pages=kw.pop("num_pages", 64),
                max_num_seqs=4, dtype=dtype, use_graph=False)
    body.update(kw)
    return ModelRunner(model_dir, EngineConfig(**body))


@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E", "F", "G", "H"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts(tmp_path, which, dtype):
    from rapid_llm_amd import StepEntry

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    pcfg, pw = plain_load(model_dir)
    runner = _runner(model_dir, dtype, page)
    gots, wants = [], []
    for i, n in enumerate([1, 5, 13, 29, 64, 100]):
        toks = random_tokens(n, cfg["vocab_size"], seed + i)
        want = plain_forward(pcfg, pw, toks)
        got = runner.step([StepEntry(f"r{i}", toks, list(range(n)))]).cpu()
        runner.finish(f"r{i}")
        if dtype == "float32":
            torch.testing.assert_close(got, want, **F32_TOL)
        else:
            gots.append(got)
            wants.append(want)
    if gots:
        parity.assert_bf16_close(torch.cat(gots), torch.cat(wants), f"whole/{which}")
    runner.cache.check_invariants()


def test_matrices_stored_in_32_bit_stay_so_in_a_bfloat16_engine(tmp_path):
    """A checkpoint may store some tensors in 32-bit: they are held and multiplied in 32-bit
    beside bfloat16 neighbours (a fused matrix with one 32-bit source is 32-bit whole), in whole
    prompts and in single decoded tokens, where the bfloat16 products around them fold norms
    into their kernels and these cannot."""
    from safetensors.torch import load_file, save_file

    from rapid_llm_amd import StepEntry

    cfg, page, seed = TINY["D"]
    model_dir = make_model_dir(tmp_path, "D", "bfloat16")
    path = str(model_dir / "model.safetensors")
    tensors = load_file(path)
    gen = torch.Generator().manual_seed(5)
    wide = ["model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight",
            "model.layers.1.self_attn.o_proj.weight", "model.layers.0.self_attn.k_proj.weight",
            "model.layers.1.mlp.down_proj.weight", "model.embed_tokens.weight"]
    for name in wide:  # values that bfloat16 cannot hold
        t = tensors[name].float()
        tensors[name] = t + 1e-4 * torch.randn(t.shape, generator=gen)
    save_file(tensors, path)
    pcfg, pw = plain_load(model_dir)
    runner = _runner(model_dir, "bfloat16", page)
    matrices = {name: p.dtype for name, p in runner.params.items() if p.dim() == 2}
    assert set(matrices.values()) == {torch.float32, torch.bfloat16}
    assert matrices["layers.0.ff.gate_up"] == torch.float32 and matrices["layers.1.ff.gate_up"] == torch.bfloat16
    assert matrices["layers.0.mixer.qkv"] == torch.float32  # one of its three sources is 32-bit
    toks = random_tokens(60, cfg["vocab_size"], seed)
    want = plain_forward(pcfg, pw, toks)
    got = [runner.step([StepEntry("r", toks[:40], list(range(40)))]).cpu()]
    for t in toks[40:]:
        got.append(runner.step([StepEntry("r", [t], [0])]).cpu())
    parity.assert_bf16_close(torch.cat(got), want, "whole/32-bit matrices beside bfloat16")
    runner.finish("r")


def test_a_bfloat16_checkpoint_in_a_float32_engine(tmp_path):
    """The engine's type, not the file's, decides the arithmetic: weights stored in bfloat16
    are widened once and everything runs in true 32-bit."""
    from rapid_llm_amd import StepEntry

    cfg, page, seed = TINY["B"]
    model_dir = make_model_dir(tmp_path, "B", "bfloat16")
    pcfg, pw = plain_load(model_dir)
    runner = _runner(model_dir, "float32", page)
    assert {p.dtype for p in runner.params.values()} == {torch.float32}
    toks = random_tokens(50, cfg["vocab_size"], seed)
    got = runner.step([StepEntry("r", toks, list(range(50)))]).cpu()
    torch.testing.assert_close(got, plain_forward(pcfg, pw, toks), **F32_TOL)
