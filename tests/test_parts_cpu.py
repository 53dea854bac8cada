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
