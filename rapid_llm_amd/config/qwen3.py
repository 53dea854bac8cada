"""The Qwen3 dense decoder's typed configuration: its ``config.json`` keys, their defaults,
what the reference fixes in code and this engine therefore refuses.
"""

from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Any, Mapping

from .model_config import ConfigError, normalise_dtype_name, read_architecture, require


@dataclass(frozen=True)
class Qwen3Config:
    """The Qwen3 dense decoder's keys (rapid_llm/models/config.py:161-294, :317-354).

    ``layer_windows[i]`` is the attention window of layer ``i`` in positions, the query's
    own included (rapid_llm/engine/kv_cache_spec.py:203-205), or 0 for all keys.
    """

    architecture: str
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    layer_windows: tuple[int, ...]
    torch_dtype: str
    eos_token_ids: tuple[int, ...]

    # ---- derived geometry (rapid_llm/models/config.py:269-294) ----------------
    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def group_size(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @classmethod
    def from_dict(
        cls, data: Mapping[str, Any], overrides: Mapping[str, Any] | None = None
    ) -> "Qwen3Config":
        data = dict(data)
        if overrides:
            data.update(overrides)  # rapid_llm/models/config.py:129-131 (hf_overrides)
        hidden = require(data, "hidden_size", int)
        layers = require(data, "num_hidden_layers", int)
        nq = require(data, "num_attention_heads", int)
        nkv = data.get("num_key_value_heads")
        if nkv is None:
            nkv = nq  # rapid_llm/models/config.py:170-173
        head_dim = data.get("head_dim")
        if head_dim is None:
            if hidden % nq:
                raise ConfigError(
                    f"hidden_size {hidden} is not divisible by num_attention_heads {nq} "
                    "and no head_dim is given"
                )
            head_dim = hidden // nq  # rapid_llm/models/config.py:175-178

        # rope_theta may sit at top level or inside the rope dict
        # (rapid_llm/models/config.py:317-335).
        theta = None
        rope_type = "default"
        for key in ("rope_parameters", "rope_scaling"):
            sub = data.get(key)
            if isinstance(sub, Mapping):
                if "rope_theta" in sub:
                    theta = sub["rope_theta"]
                rope_type = sub.get("rope_type") or sub.get("type") or rope_type
        if theta is None:
            theta = data.get("rope_theta", 10000.0)
        if rope_type not in ("default", "linear"):
            raise ConfigError(
                f"rope type {rope_type!r} is not supported for Qwen3 (only the default rotation)"
            )
        if float(data.get("partial_rotary_factor", 1.0)) != 1.0:
            raise ConfigError("partial_rotary_factor != 1.0 is not supported for Qwen3")

        # fixed in the reference's code, so anything else is refused, not ignored
        # (rapid_llm/models/qwen3.py:17, rapid_llm/modules/mlp.py:67).
        if data.get("attention_bias", False):
            raise ConfigError("attention_bias=true is not supported (Qwen3 has no q/k/v bias)")
        act = data.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act {act!r} is not supported (Qwen3 uses 'silu')")

        window = data.get("sliding_window")
        types = data.get("layer_types")
        if types is not None:
            if len(types) != layers:
                raise ConfigError(
                    f"layer_types has {len(types)} entries for {layers} layers"
                )
            windows = []
            for i, kind in enumerate(types):
                if kind == "full_attention":
                    windows.append(0)
                elif kind == "sliding_attention":
                    if not isinstance(window, int) or window < 1:
                        raise ConfigError(
                            f"layer {i} is 'sliding_attention' but sliding_window is {window!r}"
                        )
                    windows.append(window)
                else:
                    raise ConfigError(f"layer_types[{i}] = {kind!r} is not a known layer type")
        elif data.get("use_sliding_window", False):
            if not isinstance(window, int) or window < 1:
                raise ConfigError(
                    f"use_sliding_window is set but sliding_window is {window!r}"
                )
            first = data.get("max_window_layers")
            if first is None:
                first = layers
            windows = [window if i >= first else 0 for i in range(layers)]
        else:
            windows = [0] * layers

        eos = data.get("eos_token_id")
        if eos is None:
            eos_ids: tuple[int, ...] = ()
        elif isinstance(eos, int):
            eos_ids = (eos,)
        else:
            eos_ids = tuple(int(e) for e in eos)

        cfg = cls(
            architecture=read_architecture(data),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=nq,
            num_key_value_heads=int(nkv),
            head_dim=int(head_dim),
            intermediate_size=require(data, "intermediate_size", int),
            vocab_size=require(data, "vocab_size", int),
            max_position_embeddings=require(data, "max_position_embeddings", int),
            rms_norm_eps=require(data, "rms_norm_eps", float),
            rope_theta=float(theta),
            tie_word_embeddings=bool(data.get("tie_word_embeddings", False)),
            layer_windows=tuple(windows),
            torch_dtype=normalise_dtype_name(data.get("torch_dtype") or data.get("dtype") or "bfloat16"),
            eos_token_ids=eos_ids,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        """rapid_llm/models/config.py:357-388, with this engine's kernel limits."""
        for f in fields(self):
            v = getattr(self, f.name)
            if f.name in (
                "hidden_size",
                "num_hidden_layers",
                "num_attention_heads",
                "num_key_value_heads",
                "head_dim",
                "intermediate_size",
                "vocab_size",
                "max_position_embeddings",
            ) and (not isinstance(v, int) or v < 1):
                raise ConfigError(f"{f.name} must be a positive integer, got {v!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not divisible by "
                f"num_key_value_heads {self.num_key_value_heads}"
            )
        if self.head_dim % 8 or self.head_dim > 256:
            # the reference's rule (rapid_llm/models/config.py:357-388); multiples of 16 run on
            # the matrix cores, the sizes between on the slower kernel that takes any size
            raise ConfigError(
                f"head_dim {self.head_dim} is not supported: the attention kernels take "
                "multiples of 8 up to 256"
            )
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, got {self.rope_theta}")

    def to_dict(self) -> dict[str, Any]:
        """A ``config.json`` body that parses back into this configuration."""
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "torch_dtype": self.torch_dtype,
        }
        if any(self.layer_windows):
            sizes = {w for w in self.layer_windows if w}
            if len(sizes) != 1:
                raise ConfigError(
                    f"config.json has one sliding_window; layer windows {sorted(sizes)} differ"
                )
            out["sliding_window"] = sizes.pop()
            out["layer_types"] = [
                "sliding_attention" if w else "full_attention" for w in self.layer_windows
            ]
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
