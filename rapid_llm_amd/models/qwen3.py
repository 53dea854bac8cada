"""Qwen3 dense decoder: configuration -> model description, and its registry entry.

The reference's Qwen3 is two class flags on the shared skeleton, ``qkv_bias=False`` and
``use_qk_norm=True`` (rapid_llm/models/qwen3.py:16-18, rapid_llm/models/base.py:47-631).
Here it is one function that lists parts.  Checkpoint tensor names are the ones the
reference translates from (rapid_llm/models/weights.py:61-134, base.py:396-404,:493-498).
"""

from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..config.registry import register_architecture
from .spec import IgnoreRule, LayerSpec, ModelSpec, PartSpec, linear_output, token_embedding


def build_qwen3_spec(cfg: Qwen3Config) -> ModelSpec:
    rope = PartSpec(
        "rope_half_split",
        {"head_dim": cfg.head_dim, "theta": cfg.rope_theta, "rotary_dim": cfg.head_dim},
    )
    layers = []
    for i in range(cfg.num_hidden_layers):
        prefix = f"model.layers.{i}."
        layers.append(
            LayerSpec(
                mixer=PartSpec(
                    "gqa_attention",
                    {
                        "hidden_size": cfg.hidden_size,
                        "num_heads": cfg.num_attention_heads,
                        "num_kv_heads": cfg.num_key_value_heads,
                        "head_dim": cfg.head_dim,
                        "qk_norm_eps": cfg.rms_norm_eps,  # base.py:74: same eps as the layer norms
                        "window": cfg.layer_windows[i],
                        "checkpoint_prefix": prefix + "self_attn.",
                    },
                ),
                feed_forward=PartSpec(
                    "swiglu",
                    {
                        "hidden_size": cfg.hidden_size,
                        "intermediate_size": cfg.intermediate_size,
                        "checkpoint_prefix": prefix + "mlp.",
                    },
                ),
                mixer_norm=PartSpec(
                    "rmsnorm",
                    {
                        "size": cfg.hidden_size,
                        "eps": cfg.rms_norm_eps,
                        "checkpoint_name": prefix + "input_layernorm.weight",
                    },
                ),
                feed_forward_norm=PartSpec(
                    "rmsnorm",
                    {
                        "size": cfg.hidden_size,
                        "eps": cfg.rms_norm_eps,
                        "checkpoint_name": prefix + "post_attention_layernorm.weight",
                    },
                ),
                block=PartSpec("prenorm"),
                position=rope,
                checkpoint_prefix=prefix,
            )
        )
    return ModelSpec(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        layers=tuple(layers),
        final_norm=PartSpec(
            "rmsnorm",
            {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps, "checkpoint_name": "model.norm.weight"},
        ),
        embedding=token_embedding(cfg.vocab_size, cfg.hidden_size, "model.embed_tokens.weight"),
        output=linear_output(cfg.vocab_size, cfg.hidden_size, "lm_head.weight", cfg.tie_word_embeddings),
        # layers beyond num_hidden_layers are dropped unread (base.py:494-497), so a
        # layer-trimmed config.json still loads the full checkpoint
        ignore_tensors=(
            IgnoreRule(r"model\.layers\.(\d+)\..*", cfg.num_hidden_layers),
            IgnoreRule(r".*rotary_emb\.inv_freq"),
        ),
        max_position=cfg.max_position_embeddings,
    )


# Qwen3 releases that are not named "...-Base" are chat models
# (rapid_llm/utils/prompt_templates.py:96-107)
register_architecture(
    "Qwen3ForCausalLM", Qwen3Config, build_qwen3_spec, aliases=("qwen3",), replace=True, chat_by_default=True
)
