"""Weights by tensor name: coverage errors, storage types, the random-weights mode (CPU only)."""

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from rapid_llm_amd.config import Qwen3Config, resolve_architecture
from rapid_llm_amd.models import model_param_specs
from rapid_llm_amd.weights import (
    WeightsError,
    checkpoint_files,
    load_model_dir,
    load_params,
    random_checkpoint_tensors,
    write_random_model,
)
from tiny_configs import TINY_A, TINY_B, make_model_dir


def _specs(body):
    entry = resolve_architecture("Qwen3ForCausalLM")
    spec = entry.build_spec(Qwen3Config.from_dict(body))
    return spec, model_param_specs(spec)


def test_random_model_folder_loads_back_equal(tmp_path):
    folder = make_model_dir(tmp_path, "B", "float32")
    assert sorted(p.name for p in folder.iterdir()) == ["config.json", "model.safetensors"]
    body = json.loads((folder / "config.json").read_text())
    spec, specs = _specs(body)
    params = load_model_dir(folder, specs, engine_dtype=torch.float32, device="cpu",
                            ignore_rules=spec.ignore_tensors)
    stored = load_file(str(folder / "model.safetensors"))
    p = "model.layers.1.self_attn."
    fused = torch.cat([stored[p + "q_proj.weight"], stored[p + "k_proj.weight"], stored[p + "v_proj.weight"]])
    assert torch.equal(params["layers.1.mixer.qkv"], fused)  # rows [q | k | v], linear.py:253-271
    m = "model.layers.2.mlp."
    assert torch.equal(params["layers.2.ff.gate_up"], torch.cat([stored[m + "gate_proj.weight"], stored[m + "up_proj.weight"]]))
    assert torch.equal(params["final_norm.weight"], stored["model.norm.weight"])
    assert torch.equal(params["output.weight"], stored["lm_head.weight"])


def test_same_seed_same_weights_other_seed_other_weights(tmp_path):
    a = load_file(str(write_random_model(TINY_A, 5, tmp_path / "a") / "model.safetensors"))
    b = load_file(str(write_random_model(TINY_A, 5, tmp_path / "b") / "model.safetensors"))
    c = load_file(str(write_random_model(TINY_A, 6, tmp_path / "c") / "model.safetensors"))
    assert a.keys() == b.keys() == c.keys()
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert any(not torch.equal(a[k], c[k]) for k in a)
    assert "lm_head.weight" not in a  # tied: the checkpoint ships no output projection
    assert a["model.embed_tokens.weight"].dtype == torch.bfloat16  # config's torch_dtype default
    # distributions: matrices N(0, 0.02), norm weights 1 + N(0, 0.1)
    w = a["model.layers.0.mlp.gate_proj.weight"].float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    n = a["model.layers.0.input_layernorm.weight"].float()
    assert 0.7 < float(n.min()) and float(n.max()) < 1.3 and float(n.std()) > 0.03


def test_tied_output_is_the_embedding_tensor(tmp_path):
    folder = make_model_dir(tmp_path, "A", "float32")
    spec, specs = _specs(json.loads((folder / "config.json").read_text()))
    params = load_model_dir(folder, specs, engine_dtype=torch.float32, device="cpu")
    assert params["output.weight"] is params["embed.weight"]  # weights.py:197-214
    # a shipped lm_head wins over the tie
    tensors = load_file(str(folder / "model.safetensors"))
    tensors["lm_head.weight"] = torch.zeros_like(tensors["model.embed_tokens.weight"])
    save_file(tensors, str(folder / "model.safetensors"))
    params = load_model_dir(folder, specs, engine_dtype=torch.float32, device="cpu")
    assert params["output.weight"] is not params["embed.weight"]
    assert float(params["output.weight"].abs().max()) == 0.0


def test_storage_types(tmp_path):
    spec, specs = _specs(TINY_B)
    tensors = random_checkpoint_tensors(specs, 1, dtype="bfloat16")
    tensors["model.layers.0.mlp.down_proj.weight"] = tensors["model.layers.0.mlp.down_proj.weight"].float()
    bf = load_params(specs, tensors.items(), engine_dtype=torch.bfloat16, device="cpu")
    assert bf["layers.1.ff.down"].dtype == torch.bfloat16
    assert bf["layers.0.ff.down"].dtype == torch.float32  # stored in 32-bit, stays so
    assert bf["layers.0.mixer_norm.weight"].dtype == torch.float32  # vectors are held in float32
    f32 = load_params(specs, tensors.items(), engine_dtype=torch.float32, device="cpu")
    assert all(t.dtype == torch.float32 for t in f32.values())


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    spec, specs = _specs(TINY_B)
    tensors = random_checkpoint_tensors(specs, 1, dtype="float32")
    del tensors["model.layers.1.self_attn.k_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary_bias"] = torch.zeros(3)
    tensors["model.layers.2.mlp.up_proj.weight"] = torch.zeros(7, 96)
    tensors["lm_head.weight"] = torch.zeros(503, 95)
    with pytest.raises(WeightsError) as err:
        load_params(specs, tensors.items(), engine_dtype=torch.float32, device="cpu",
                    ignore_rules=spec.ignore_tensors, where="unit test")
    e = err.value
    assert [m.split()[0] for m in e.missing] == ["model.layers.1.self_attn.k_proj.weight", "model.norm.weight"]
    assert [u.split()[0] for u in e.unexpected] == ["model.layers.0.self_attn.rotary_bias"]
    assert sorted(w.split(":")[0] for w in e.wrong_shape) == ["lm_head.weight", "model.layers.2.mlp.up_proj.weight"]
    text = str(e)
    assert "unit test" in text and "(7, 96)" in text and "(320, 96)" in text and "layers.1.mixer.qkv" in text


def test_untied_model_without_output_projection_is_an_error():
    spec, specs = _specs(TINY_B)
    tensors = random_checkpoint_tensors(specs, 1, dtype="float32")
    del tensors["lm_head.weight"]
    with pytest.raises(WeightsError, match="lm_head.weight"):
        load_params(specs, tensors.items(), engine_dtype=torch.float32, device="cpu")


def test_layers_beyond_the_configuration_are_dropped_unread():
    spec, specs = _specs(dict(TINY_B, num_hidden_layers=2))  # base.py:494-497
    full = random_checkpoint_tensors(_specs(TINY_B)[1], 1, dtype="float32")
    full["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    params = load_params(specs, full.items(), engine_dtype=torch.float32, device="cpu",
                         ignore_rules=spec.ignore_tensors)
    assert "layers.1.ff.down" in params and "layers.2.ff.down" not in params


def test_duplicate_and_non_float_tensors():
    spec, specs = _specs(TINY_A)
    tensors = random_checkpoint_tensors(specs, 1, dtype="float32")
    items = list(tensors.items()) + [("model.norm.weight", tensors["model.norm.weight"])]
    with pytest.raises(WeightsError, match="appears twice"):
        load_params(specs, items, engine_dtype=torch.float32, device="cpu")
    tensors["model.norm.weight"] = tensors["model.norm.weight"].to(torch.int64)
    with pytest.raises(WeightsError, match="does not load"):
        load_params(specs, tensors.items(), engine_dtype=torch.float32, device="cpu")


def test_empty_folder_names_what_it_wanted(tmp_path):
    with pytest.raises(FileNotFoundError, match="safetensors"):
        checkpoint_files(tmp_path)
