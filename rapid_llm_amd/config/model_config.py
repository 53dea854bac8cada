"""What every typed model configuration shares: reading ``config.json`` with ``json`` alone,
finding the architecture's name in it, the storage types, the errors.

A configuration class owns the names of its architecture's keys and their defaults; no size
and no constant that ``config.json`` gives appears anywhere else in the package.  Each
architecture's class lives in a file of its own beside this one (``config/qwen3.py``) and is
named in that architecture's registry entry.  The reference wraps ``transformers.AutoConfig``
(rapid_llm/models/config.py:111-132) and normalises geometry through properties (:161-294);
here one frozen dataclass per architecture does both.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping


class ConfigError(ValueError):
    """A ``config.json`` that is missing, malformed, or asks for something unsupported."""


def read_config_json(model_dir: str | Path) -> dict[str, Any]:
    """Read ``<model_dir>/config.json``.

    Same three failures as rapid_llm/models/config.py:42-62: no file, not JSON, not an object.
    """
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json under {str(model_dir)!r}")
    try:
        data = json.loads(path.read_text())
    except json.JSONDecodeError as exc:
        raise ConfigError(f"{path} is not valid JSON: {exc}") from exc
    if not isinstance(data, dict):
        raise ConfigError(f"{path} must hold a JSON object, got {type(data).__name__}")
    return data


def read_architecture(data: Mapping[str, Any]) -> str:
    """The registry key of a configuration: ``architectures[0]``, else ``model_type``.

    The reference keys its registry on ``model_type`` (rapid_llm/models/registry.py:44-78);
    both spellings are accepted here and resolved by the registry.
    """
    archs = data.get("architectures")
    if isinstance(archs, (list, tuple)) and archs and isinstance(archs[0], str):
        return archs[0]
    model_type = data.get("model_type")
    if isinstance(model_type, str) and model_type:
        return model_type
    raise ConfigError("config.json names neither 'architectures' nor 'model_type'")


_DTYPE_NAMES = {
    "float32": "float32",
    "fp32": "float32",
    "float": "float32",
    "bfloat16": "bfloat16",
    "bf16": "bfloat16",
}


def normalise_dtype_name(name: str) -> str:
    try:
        return _DTYPE_NAMES[str(name).lower().replace("torch.", "")]
    except KeyError:
        raise ConfigError(
            f"unsupported dtype {name!r}; this engine runs 'bfloat16' and 'float32'"
        ) from None


def require(data: Mapping[str, Any], key: str, kind: type) -> Any:
    if key not in data or data[key] is None:
        raise ConfigError(f"config.json lacks the required key {key!r}")
    value = data[key]
    if kind is float and isinstance(value, int) and not isinstance(value, bool):
        value = float(value)
    if not isinstance(value, kind) or isinstance(value, bool) and kind is not bool:
        raise ConfigError(f"config.json key {key!r} must be {kind.__name__}, got {value!r}")
    return value
