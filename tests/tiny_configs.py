"""Tiny configurations of the Qwen3 dense decoder that differ in every size and option."""

import random
from pathlib import Path

# A: tied embeddings, group 2, head 16, power-of-two sizes, small page
TINY_A = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
    head_dim=16, intermediate_size=128, vocab_size=256, rope_theta=10000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=128,
    hidden_act="silu", attention_bias=False,
)
PAGE_A = 4

# B: untied, one kv head (group 6), head 32 with heads*head_dim != hidden, odd vocabulary
TINY_B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=1,
    head_dim=32, intermediate_size=320, vocab_size=503, rope_theta=1000000.0,
    rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=256,
    hidden_act="silu", attention_bias=False,
)
PAGE_B = 16

# C: windowed layers beside a full one (two cache groups), head 48 (no power of two),
# as many kv heads as query heads, width 80, vocabulary 331
TINY_C = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=3, hidden_size=80, num_attention_heads=5, num_key_value_heads=5,
    head_dim=48, intermediate_size=176, vocab_size=331, rope_theta=500000.0,
    rms_norm_eps=3e-6, tie_word_embeddings=False, max_position_embeddings=512,
    hidden_act="silu", attention_bias=False,
    sliding_window=21, layer_types=["full_attention", "sliding_attention", "sliding_attention"],
)
PAGE_C = 8

# D: head 64 (the size from which a decode step's norm, rotation, cache write and attention
# run as one kernel), a window on the last layer, group 3, page 8
TINY_D = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=112, num_attention_heads=6, num_key_value_heads=2,
    head_dim=64, intermediate_size=200, vocab_size=389, rope_theta=250000.0,
    rms_norm_eps=2e-6, tie_word_embeddings=True, max_position_embeddings=640,
    hidden_act="silu", attention_bias=False,
    sliding_window=150, layer_types=["full_attention", "sliding_attention"],
)
PAGE_D = 8

# E: widths that are multiples of 128, which the product for 17 to 64 rows needs (the output
# projection in one run of K, the down projection in two), group 2, head 32, page 8
TINY_E = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=128, num_attention_heads=4, num_key_value_heads=2,
    head_dim=32, intermediate_size=1024, vocab_size=277, rope_theta=30000.0,
    rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=256,
    hidden_act="silu", attention_bias=False,
)
PAGE_E = 8
# F: widths that no vector access divides (70 = 2 * 35, 99 odd, vocabulary 211 prime): every
# kernel takes its element-by-element path and the bfloat16 products go to the library;
# heads * head_dim = 96 beside a width of 70; a page larger than most requests
TINY_F = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=70, num_attention_heads=6, num_key_value_heads=3,
    head_dim=16, intermediate_size=99, vocab_size=211, rope_theta=7777.0,
    rms_norm_eps=4e-6, tie_word_embeddings=False, max_position_embeddings=256,
    hidden_act="silu", attention_bias=False,
)
PAGE_F = 32

# G: a head size between the matrix cores' steps of 16 (24: the kernel that takes any size runs
# the attention, in both types), group 3, a window on the first layer, vocabulary 257, page 4
TINY_G = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=88, num_attention_heads=3, num_key_value_heads=1,
    head_dim=24, intermediate_size=136, vocab_size=257, rope_theta=40000.0,
    rms_norm_eps=5e-6, tie_word_embeddings=True, max_position_embeddings=192,
    hidden_act="silu", attention_bias=False,
    sliding_window=37, layer_types=["sliding_attention", "full_attention"],
)
PAGE_G = 4

# H: head 128, the family's own: from this size on a prompt step's key and value tiles go from
# memory straight into LDS, and the attention kernels finish the query heads' norm and rotation
# themselves; a window on the first layer, group 2, heads * head_dim = 512 beside a width of 192
TINY_H = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3",
    num_hidden_layers=2, hidden_size=192, num_attention_heads=4, num_key_value_heads=2,
    head_dim=128, intermediate_size=272, vocab_size=401, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=640,
    hidden_act="silu", attention_bias=False,
    sliding_window=70, layer_types=["sliding_attention", "full_attention"],
)
PAGE_H = 16

TINY = {"H": (TINY_H, PAGE_H, 88), "A": (TINY_A, PAGE_A, 11), "B": (TINY_B, PAGE_B, 22), "C": (TINY_C, PAGE_C, 33),
        "D": (TINY_D, PAGE_D, 44), "E": (TINY_E, PAGE_E, 55), "F": (TINY_F, PAGE_F, 66),
        "G": (TINY_G, PAGE_G, 77)}


def make_model_dir(tmp_path: Path, which: str, dtype: str = "float32") -> Path:
    """Write config.json + model.safetensors of a tiny model (norm weights 1 + N(0, 0.1))."""
    from rapid_llm_amd.weights import write_random_model

    cfg, _page, seed = TINY[which]
    out = Path(tmp_path) / f"tiny_{which}_{dtype}"
    write_random_model(dict(cfg), seed, out, dtype=dtype, norm_std=0.1)
    return out


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]
