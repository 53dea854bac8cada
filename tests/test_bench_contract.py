"""What the measurement's figures are made of (CPU only): the bytes of a decode step and the
flops of a prompt step for the benchmark's shape, and the refusal of more than one GPU."""

import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))


def _shape():
    import bench

    from rapid_llm_amd.config import Qwen3Config

    shape = bench.load_shape()
    context, prompt_len = shape.pop("context"), shape.pop("prompt_len")
    return bench, Qwen3Config.from_dict(shape), context, prompt_len


def test_the_default_shape_is_the_one_the_baseline_names():
    bench, cfg, context, prompt_len = _shape()
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (36, 4096, 32, 8)
    assert (cfg.head_dim, cfg.intermediate_size, cfg.vocab_size, cfg.tie_word_embeddings) == (128, 12288, 151936, False)
    assert (context, prompt_len) == (4096, 2048)


def test_bytes_of_a_decode_step_and_flops_of_a_prompt_step():
    """Every weight a step uses once (the embedding table is not one of them: a step reads a
    row of it a token) and the cache of the live requests; a prompt's flops are two a
    multiply-add of every product, the attention's causal half, one row of logits."""
    bench, cfg, _, _ = _shape()
    per_layer = 6144 * 4096 + 4096 * 4096 + 24576 * 4096 + 4096 * 12288
    assert bench.weight_bytes(cfg, 2) == (36 * per_layer + 151936 * 4096) * 2  # 15.14 GB
    assert abs(bench.weight_bytes(cfg, 2) / 1e9 - 15.14) < 0.01
    assert bench.kv_bytes_per_token(cfg, 2) == 2 * 8 * 128 * 36 * 2 == 147456
    flops = bench.prefill_flops(cfg, 2048)
    linear = 2.0 * 2048 * per_layer * 36
    attention = 4.0 * 4096 * (2048 * 2049 / 2) * 36
    assert abs(flops - (linear + attention + 2.0 * 151936 * 4096)) < 1e6
    assert 29.0e12 < flops < 30.5e12
    assert bench.HBM_GBPS == 8000.0 and bench.PEAK_TFLOPS == {"bfloat16": 2500.0, "float32": 157.3}


def test_more_than_one_gpu_is_one_line_and_exit_code_2():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert done.returncode == 2
    assert len(done.stdout.strip().splitlines()) == 1 and "one GPU" in done.stdout
