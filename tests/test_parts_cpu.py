"""What parts decide on the host, without a device."""

import torch

from rapid_llm_amd.parts.linear import Linear


def _bound(in_features, out_features, dtype):
    linear = Linear(in_features, out_features)
    linear.bind(torch.zeros(out_features, in_features, dtype=dtype))
    return linear


def test_a_product_takes_unscaled_rows_only_if_its_few_row_kernel_runs():
    """A norm leaves its factor to the product behind it only where that product's kernel can
    apply it: bfloat16 weights and a width the kernel's 16-byte reads divide.  A width of 70
    behind an output projection of width 96 once reached the library product with rows that
    nobody had scaled."""
    assert _bound(96, 70, torch.bfloat16).takes_scaled_rows()
    assert not _bound(70, 198, torch.bfloat16).takes_scaled_rows()
    assert not _bound(96, 70, torch.float32).takes_scaled_rows()  # a matrix the checkpoint stores in 32-bit
    assert not Linear(96, 70).takes_scaled_rows()  # nothing bound yet


class _ByteTokenizer:
    """Token id = one byte: a character of several bytes spans tokens."""

    def decode(self, ids, skip_special_tokens=True):
        return bytes(ids).decode("utf-8", errors="replace")


def test_text_is_released_only_with_whole_characters():
    from rapid_llm_amd.engine.tokenizer import Detokenizer

    text = "a é 漢字 ok"
    detok = Detokenizer(_ByteTokenizer())
    pieces = [detok.append(b) for b in text.encode("utf-8")]
    assert "".join(pieces) == text
    assert all("�" not in p for p in pieces)
    assert pieces[2] == "" and pieces[3] == "é"  # the first byte of a two-byte character releases nothing


def test_stop_ids_come_from_generation_config_and_config(tmp_path):
    from rapid_llm_amd.engine.tokenizer import load_stop_token_ids, load_tokenizer

    assert load_stop_token_ids(tmp_path, config_eos=[7]) == {7}
    (tmp_path / "generation_config.json").write_text('{"eos_token_id": [3, 9]}')
    assert load_stop_token_ids(tmp_path, config_eos=[7]) == {3, 7, 9}
    (tmp_path / "generation_config.json").write_text('{"eos_token_id": 4}')
    assert load_stop_token_ids(tmp_path) == {4}
    (tmp_path / "generation_config.json").write_text("{not json")
    assert load_stop_token_ids(tmp_path, config_eos=[1]) == {1}
    assert load_tokenizer(tmp_path) is None  # no tokenizer.json: prompts are token ids


def test_command_line_init_writes_a_model_folder_and_names_a_missing_one(tmp_path, capsys, monkeypatch):
    import json

    import pytest
    from safetensors.torch import load_file

    from rapid_llm_amd.cli import main
    from tiny_configs import TINY_B

    config = tmp_path / "config.json"
    config.write_text(json.dumps(TINY_B))
    for seed in (4, 4, 5):
        assert main(["init", "--config", str(config), "--out", str(tmp_path / f"m{seed}"), "--seed", str(seed),
                     "--dtype", "bfloat16"]) == 0
    a = load_file(str(tmp_path / "m4" / "model.safetensors"))
    assert json.loads((tmp_path / "m4" / "config.json").read_text())["torch_dtype"] == "bfloat16"
    assert a["model.layers.2.mlp.down_proj.weight"].shape == (96, 320)
    assert a["model.embed_tokens.weight"].dtype == __import__("torch").bfloat16
    b = load_file(str(tmp_path / "m5" / "model.safetensors"))
    assert not (a["lm_head.weight"] == b["lm_head.weight"]).all()
    # generation commands name the folder they lack, or take it from the environment
    monkeypatch.delenv("RAPID_LLM_MODEL_DIR", raising=False)
    with pytest.raises(SystemExit, match="Model directory not provided"):
        main(["batch"])
    monkeypatch.setenv("RAPID_LLM_MODEL_DIR", str(tmp_path / "nowhere"))
    with pytest.raises(SystemExit, match="does not exist"):
        main(["batch"])


def test_a_product_with_a_bias_folds_no_norm_into_itself():
    """The residual add and norm that follow a product are folded into its kernel only where
    nothing comes between: a bias is added by a kernel of its own after the product."""
    plain = _bound(128, 128, torch.bfloat16)
    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    assert plain.folds(x) and plain.folds(torch.zeros(40, 128, dtype=torch.bfloat16))
    assert plain.folds(torch.zeros(192, 128, dtype=torch.bfloat16))  # runs of K, in blocks of 64 rows
    assert not plain.folds(torch.zeros(193, 128, dtype=torch.bfloat16))  # the library's product
    biased = Linear(128, 128)
    biased.bind(torch.zeros(128, 128, dtype=torch.bfloat16), torch.zeros(128))
    assert not biased.folds(x) and biased.skinny(x)
    import pytest

    with pytest.raises(ValueError, match="bias"):
        Linear(128, 64).bind(torch.zeros(64, 128, dtype=torch.bfloat16), torch.zeros(128))
    with pytest.raises(ValueError, match="bias"):
        Linear(128, 64).bind(torch.zeros(64, 128, dtype=torch.bfloat16), torch.zeros(64, dtype=torch.bfloat16))


def test_a_mixer_may_ask_for_several_state_tensors():
    import pytest

    from rapid_llm_amd.cache.storage import state_bytes
    from rapid_llm_amd.parts import CacheNeed, StateSpec

    one = CacheNeed("state", state_shape=(48,), state_dtype="float32")
    assert [(s.name, s.shape, s.dtype) for s in one.state_specs()] == [("state", (48,), "float32")]
    two = CacheNeed.keys_and_values(2, 16,
                    states=(StateSpec("conv", (3, 48)), StateSpec("count", (1,), "int32")))
    assert [s.name for s in two.state_specs()] == ["conv", "count"]
    assert CacheNeed.keys_and_values(1, 16).state_specs() == ()
    # five slots: 48 float32 each; 3 x 48 in the engine's type (2 bytes) and one int32 each
    assert state_bytes([one, two], 5, 2) == 5 * 48 * 4 + 5 * (3 * 48 * 2 + 4)
    with pytest.raises(ValueError, match="alike"):
        CacheNeed("state", state_shape=(4,), states=(StateSpec("state", (2,)),)).state_specs()


def test_the_ends_of_a_model_are_parts_named_in_its_description():
    from rapid_llm_amd.models import linear_output, token_embedding
    from rapid_llm_amd.parts import EMBEDDINGS, OUTPUT_PROJECTIONS

    assert "token_embedding" in EMBEDDINGS.kinds() and "linear_output" in OUTPUT_PROJECTIONS.kinds()
    emb = token_embedding(100, 16, "model.embed_tokens.weight")
    part = EMBEDDINGS.create(emb.kind, **emb.params, name="embed")
    assert [(s.name, s.shape) for s in part.param_specs()] == [("embed.weight", (100, 16))]
    tied = linear_output(100, 16, "lm_head.weight", True)
    out = OUTPUT_PROJECTIONS.create(tied.kind, **tied.params, name="output")
    assert out.param_specs()[0].fallback == "embed.weight"
    assert OUTPUT_PROJECTIONS.create("linear_output", **linear_output(100, 16, "h", False).params, name="output").param_specs()[0].fallback is None


def test_prefill_launch_shapes_follow_an_estimate_of_the_launch():
    """Two wave groups on a tile where the longest tile would outlast everyone else's work (a
    prompt from its start), one where there is work for every slot, key runs for few, long tiles
    and only where they save more than their merge costs.  The choice is the host's alone."""
    from types import SimpleNamespace

    from rapid_llm_amd.kernels import ops

    def shape(seqs, nkv=8, group=4, window=0, rows=128):
        keys = []
        for start, n in seqs:
            for row0 in range(0, n * group, rows):
                keys.append(start + min(n, (row0 + rows) // group))
        return ops._prefill_shape(SimpleNamespace(tile_keys=keys, num_tiles=len(keys)), nkv, window, rows)

    assert shape([(0, 2048)]) == (2, 1) and shape([(0, 1024)]) == (2, 1) and shape([(0, 512)]) == (2, 1)
    assert shape([(0, 8192)]) == (1, 1) and shape([(0, 4096)]) == (1, 1) and shape([(2048, 2048)]) == (1, 1)
    assert shape([(3584, 512)]) == (1, 4) and shape([(7680, 512)]) == (1, 4) and shape([(16000, 150)]) == (1, 8)
    assert shape([(0, 2048)] * 4) == (1, 1) and shape([(0, 20)]) == (1, 1)
    # a window bounds what every tile reads: the long prefix no longer counts
    assert shape([(16000, 150)], window=256) == (2, 1)


def test_which_products_run_in_one_launch_of_this_package():
    """The host's rule for the tile product (17 to 512 rows over a matrix of a few megabytes with
    enough result columns for every compute unit): the smallest model's QKV and gate/up products
    take it, its narrow products, larger models' matrices and steps of few or many rows do not."""
    from rapid_llm_amd.kernels import ops

    assert ops._tile_applies(64, 4096, 1024, 4096)        # Qwen3-0.6B QKV
    assert ops._tile_applies(256, 6144, 1024, 3072)       # its packed gate and up rows, 3,072 results
    assert ops._tile_applies(512, 4096, 1024, 4096)
    assert not ops._tile_applies(16, 4096, 1024, 4096)    # the few-row kernel's
    assert not ops._tile_applies(513, 4096, 1024, 4096)   # the library's
    assert not ops._tile_applies(64, 1024, 2048, 1024)    # output projection: 16 workgroups a row block
    assert not ops._tile_applies(64, 4096, 2048, 4096)    # 16 MB: the library is as fast
    assert not ops._tile_applies(64, 6144, 4096, 6144)    # Qwen3-8B QKV
    assert not ops._tile_applies(64, 4096, 1000, 4096)    # K in chunks of 128 only
    assert not ops._tile_applies(64, 4098, 1024, 4098)    # four result columns a lane


def test_launch_rules_follow_the_number_of_compute_units():
    """Every launch rule takes the chip's geometry from one place on the host
    (``ops.chip()``; without a device the chip the rules were measured on), so that a part
    with another number of compute units gets shapes for itself: decode attention asks for the
    requests' order by length only beyond three workgroups a unit, and the few-row product's
    rows a workgroup and the runs of K of the mid-size product move with the unit count."""
    from types import SimpleNamespace

    from rapid_llm_amd.kernels import ops

    assert ops.chip().units == 256 and ops.chip().decode_resident == 3 * 256
    assert ops.Chip(304).first_round == 304 and ops.Chip(304).prefill_slots == 608
    # 384 tiles of 16 rows: one round of 24 rows on 256 units, nothing to gain on 384 units
    assert ops._skinny_tiles(8, 6144, plain=True, units=256) == 3
    assert ops._skinny_tiles(8, 6144, plain=True, units=384) == 1
    # 64 blocks of 64 rows: four runs of K fill 256 units, one run fills 64
    assert ops.mid_runs(4096, 4096, units=256) == 4 and ops.mid_runs(4096, 4096, units=64) == 1
    # a portion behind a long prefix is cut into key runs only while the launch leaves slots free
    tile = SimpleNamespace(tile_keys=[4096] * 4, num_tiles=4)
    assert ops._prefill_shape(tile, 8, 0, 128, units=256)[1] > 1
    assert ops._prefill_shape(tile, 8, 0, 128, units=8) == (1, 1)


def test_weight_rows_a_workgroup_of_the_few_row_product():
    """The host's rule: 24 rows (code 3) only for a product that just stores its result, on a
    matrix of 257 to 1,023 tiles, where that puts the fewest rows on a compute unit."""
    from rapid_llm_amd.kernels import ops

    assert ops._skinny_tiles(8, 6144, plain=True) == 3      # 384 tiles: 256 workgroups of 24 rows
    assert ops._skinny_tiles(1, 5120, plain=True) == 3      # 320 tiles: 214 workgroups
    assert ops._skinny_tiles(8, 7168, plain=True) == 2      # 448 tiles: 24 rows would need a second round
    assert ops._skinny_tiles(8, 6144) == 2                  # the residual epilogue keeps whole tiles
    assert ops._skinny_tiles(8, 4096, plain=True) == 1      # one tile a unit already
    assert ops._skinny_tiles(16, 151936, plain=True) == 2   # a thousand tiles and more: as measured
    assert ops._skinny_tiles(8, 151936, plain=True) == 1


def test_tiles_a_workgroup_of_the_product_for_tens_of_rows():
    """The host's rule for the product of 17 to 64 rows over wide matrices: a compute unit gets
    one workgroup with an even share of the tiles where a workgroup can hold such a share, and a
    matrix with more tiles is cut into workgroups of the most tiles one holds."""
    from rapid_llm_amd.kernels import ops

    plan = lambda m, n, k, sw: ops.rows_plan(m, n, k, sw, units=256)
    assert plan(64, 12288, 4096, True) == (3, 256)     # Qwen3-8B gate/up: 768 pairs, three a unit
    assert plan(32, 6144, 4096, False) == (2, 256)     # its QKV: 384 tiles, one or two a unit
    assert plan(64, 151936, 4096, False) == (6, 1583)  # the vocabulary: 9,496 tiles in groups of six
    assert plan(48, 25600, 5120, True) is None         # the 32B shape's gate/up, 1,600 pairs: the library's,
    assert plan(48, 51200, 5120, False) is None        # with the activation or without
    assert plan(33, 17408, 5120, True) == (5, 256) and plan(33, 10240, 5120, False) == (3, 256)
    assert plan(64, 17408, 5120, True) == (3, 363)     # at 64 rows a workgroup holds three pairs at most
    assert plan(33, 4096, 2048, False) == (1, 256) and plan(33, 2048, 2048, False) == (1, 128)
    assert plan(33, 12288, 4096, True) == (3, 256) and ops.rows_plan(33, 12288, 4096, True, units=304) == (3, 304)
    assert plan(16, 12288, 4096, True) is None and plan(65, 12288, 4096, True) is None
    assert plan(33, 12296, 4096, True) is None and plan(33, 12288, 4160, True) is None
