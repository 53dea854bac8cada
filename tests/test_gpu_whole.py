"""Each request alone and whole, float32 and bfloat16, against the plain implementation."""

import pytest
import torch

from plain_model import plain_forward, plain_load
from tiny_configs import TINY, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

F32_TOL = dict(rtol=2e-5, atol=3e-6)
BF16_TOL = dict(rtol=5e-2, atol=3e-2)


def _runner(model_dir, dtype, page, **kw):
    from rapid_llm_amd import EngineConfig, ModelRunner

    body = dict(max_seq_len=kw.pop("max_seq_len", 128), page_size=page, num_pages=kw.pop("num_pages", 64),
                max_num_seqs=4, dtype=dtype, use_graph=False)
    body.update(kw)
    return ModelRunner(model_dir, EngineConfig(**body))


@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E", "F"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts(tmp_path, which, dtype):
    from rapid_llm_amd import StepEntry

    cfg, page, seed = TINY[which]
    model_dir = make_model_dir(tmp_path, which, dtype)
    pcfg, pw = plain_load(model_dir)
    runner = _runner(model_dir, dtype, page)
    for i, n in enumerate([1, 5, 13, 29, 64, 100]):
        toks = random_tokens(n, cfg["vocab_size"], seed + i)
        want = plain_forward(pcfg, pw, toks)
        got = runner.step([StepEntry(f"r{i}", toks, list(range(n)))]).cpu()
        runner.finish(f"r{i}")
        tol = F32_TOL if dtype == "float32" else BF16_TOL
        torch.testing.assert_close(got, want, **tol)
    runner.cache.check_invariants()
