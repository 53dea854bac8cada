"""Typed configuration and the architecture registry (CPU only)."""

import json

import pytest

from rapid_llm_amd.config import (
    ConfigError,
    EngineConfig,
    Qwen3Config,
    config_from_dict,
    read_architecture,
    read_config_json,
    register_architecture,
    resolve_architecture,
    supported_architectures,
    unregister_architecture,
)
from tiny_configs import TINY_A, TINY_B, TINY_C


def test_every_key_is_read_from_config_json():
    cfg = Qwen3Config.from_dict(TINY_B)
    assert (cfg.hidden_size, cfg.num_hidden_layers, cfg.num_attention_heads) == (96, 3, 6)
    assert (cfg.num_key_value_heads, cfg.head_dim, cfg.intermediate_size) == (1, 32, 320)
    assert (cfg.vocab_size, cfg.max_position_embeddings) == (503, 256)
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 1e6
    assert cfg.tie_word_embeddings is False
    assert cfg.q_size == 192 and cfg.kv_size == 32 and cfg.group_size == 6
    assert cfg.layer_windows == (0, 0, 0)


def test_defaults_of_the_reference():
    body = dict(TINY_A)
    del body["num_key_value_heads"], body["head_dim"], body["rope_theta"]
    cfg = Qwen3Config.from_dict(body)
    assert cfg.num_key_value_heads == cfg.num_attention_heads  # config.py:170-173
    assert cfg.head_dim == 64 // 4  # config.py:175-178
    assert cfg.rope_theta == 10000.0  # config.py:317-335


def test_rope_theta_inside_rope_parameters():
    body = dict(TINY_A, rope_parameters={"rope_theta": 12345.0, "rope_type": "default"})
    del body["rope_theta"]
    assert Qwen3Config.from_dict(body).rope_theta == 12345.0


def test_round_trip_through_config_json(tmp_path):
    for body in (TINY_A, TINY_B, TINY_C):
        cfg = Qwen3Config.from_dict(body)
        (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
        entry, again = config_from_dict(read_config_json(tmp_path))
        assert again == cfg
        assert entry.name == "Qwen3ForCausalLM"


def test_window_keys():
    cfg = Qwen3Config.from_dict(TINY_C)
    assert cfg.layer_windows == (0, 21, 21)
    body = dict(TINY_A, use_sliding_window=True, sliding_window=8, max_window_layers=1)
    assert Qwen3Config.from_dict(body).layer_windows == (0, 8)
    with pytest.raises(ConfigError, match="sliding_window"):
        Qwen3Config.from_dict(dict(TINY_A, layer_types=["sliding_attention", "full_attention"]))
    with pytest.raises(ConfigError, match="layer_types has 1"):
        Qwen3Config.from_dict(dict(TINY_A, layer_types=["full_attention"]))


@pytest.mark.parametrize(
    "change, message",
    [
        ({"hidden_size": None}, "hidden_size"),
        ({"rms_norm_eps": None}, "rms_norm_eps"),
        ({"num_attention_heads": 3}, "not divisible"),
        ({"head_dim": 20}, "head_dim 20"),
        ({"head_dim": 272}, "head_dim 272"),
        ({"attention_bias": True}, "attention_bias"),
        ({"hidden_act": "gelu"}, "hidden_act"),
        ({"rope_scaling": {"rope_type": "yarn", "factor": 4.0}}, "rope type"),
        ({"partial_rotary_factor": 0.5}, "partial_rotary_factor"),
        ({"vocab_size": 0}, "vocab_size"),
        ({"torch_dtype": "float16"}, "dtype"),
        ({"num_hidden_layers": "2"}, "num_hidden_layers"),
    ],
)
def test_what_is_refused(change, message):
    with pytest.raises(ConfigError, match=message):
        Qwen3Config.from_dict(dict(TINY_A, **change))


def test_read_config_json_failures(tmp_path):
    with pytest.raises(FileNotFoundError):
        read_config_json(tmp_path)
    (tmp_path / "config.json").write_text("{ not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        read_config_json(tmp_path)
    (tmp_path / "config.json").write_text("[1, 2]")
    with pytest.raises(ConfigError, match="JSON object"):
        read_config_json(tmp_path)
    with pytest.raises(ConfigError, match="neither"):
        read_architecture({"hidden_size": 4})


def test_registry_resolves_both_spellings_and_lists_alternatives():
    assert resolve_architecture("Qwen3ForCausalLM") is resolve_architecture("qwen3")
    assert "Qwen3ForCausalLM" in supported_architectures()
    with pytest.raises(ConfigError, match="supported: .*Qwen3ForCausalLM"):
        resolve_architecture("NoSuchModel")


def test_another_architecture_is_one_call():
    class ToyConfig:
        @classmethod
        def from_dict(cls, data, overrides=None):
            return cls()

    try:
        register_architecture("ToyForCausalLM", ToyConfig, lambda cfg: "spec", aliases=("toy",))
        with pytest.raises(ValueError, match="already registered"):
            register_architecture("ToyForCausalLM", ToyConfig, lambda cfg: "spec")
        entry, cfg = config_from_dict({"architectures": ["ToyForCausalLM"]})
        assert isinstance(cfg, ToyConfig) and entry.build_spec(cfg) == "spec"
        assert config_from_dict({"model_type": "toy"})[0] is entry
    finally:
        unregister_architecture("ToyForCausalLM")
    with pytest.raises(ConfigError):
        resolve_architecture("toy")


def test_engine_config_validation():
    EngineConfig()
    for bad in (
        dict(max_seq_len=1),
        dict(page_size=6),
        dict(max_num_seqs=0),
        dict(max_num_batched_tokens=0),
        dict(max_chunk_size=-1),
        dict(max_chunk_size=0, max_num_batched_tokens=100, max_seq_len=2048),
        dict(num_pages=1),
        dict(gpu_memory_utilization=0.0),
        dict(dtype="float16"),
    ):
        with pytest.raises(ConfigError):
            EngineConfig(**bad)
    assert EngineConfig(dtype="bf16").dtype == "bfloat16"


def test_spec_holds_no_size_of_its_own():
    """The model description is made of the configuration's numbers alone."""
    entry = resolve_architecture("Qwen3ForCausalLM")
    for body in (TINY_A, TINY_B, TINY_C):
        cfg = Qwen3Config.from_dict(body)
        spec = entry.build_spec(cfg)
        assert len(spec.layers) == cfg.num_hidden_layers
        assert spec.vocab_size == cfg.vocab_size and spec.hidden_size == cfg.hidden_size
        for i, layer in enumerate(spec.layers):
            m = layer.mixer.params
            assert (m["num_heads"], m["num_kv_heads"], m["head_dim"]) == (
                cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim)
            assert m["window"] == cfg.layer_windows[i]
            assert m["qk_norm_eps"] == cfg.rms_norm_eps
            assert layer.feed_forward.params["intermediate_size"] == cfg.intermediate_size
            assert layer.mixer_norm.params["eps"] == cfg.rms_norm_eps
            assert layer.position.params["theta"] == cfg.rope_theta
