"""One registry: architecture name -> (configuration class, model description builder).

The reference maps ``model_type`` to a lazily imported ``"module:Class"``
(rapid_llm/models/registry.py:20-78) and raises listing the alternatives (:69-78).
Here an entry names the typed configuration that parses ``config.json`` and the function
that turns that configuration into a :class:`~rapid_llm_amd.models.spec.ModelSpec`, the
pure-data description the generic model is built from.  Adding an architecture is one
``register_architecture`` call; nothing else in the package names an architecture.
"""

from __future__ import annotations

import importlib
from dataclasses import dataclass
from typing import Any, Callable, Mapping

from .model_config import ConfigError, read_architecture


@dataclass(frozen=True)
class ArchitectureEntry:
    name: str
    config_cls: Any  # has from_dict(data, overrides) and to_dict()
    build_spec: Callable[[Any], Any]  # config -> ModelSpec
    aliases: tuple[str, ...] = ()


_ENTRIES: dict[str, ArchitectureEntry] = {}
_ALIASES: dict[str, str] = {}
# built-in architectures, imported on first lookup so that importing the package stays cheap
_LAZY: dict[str, str] = {
    "Qwen3ForCausalLM": "rapid_llm_amd.models.qwen3",
    "qwen3": "rapid_llm_amd.models.qwen3",
}


def register_architecture(
    name: str,
    config_cls: Any,
    build_spec: Callable[[Any], Any],
    aliases: tuple[str, ...] = (),
    *,
    replace: bool = False,
) -> ArchitectureEntry:
    if name in _ENTRIES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    entry = ArchitectureEntry(name, config_cls, build_spec, tuple(aliases))
    _ENTRIES[name] = entry
    for alias in aliases:
        _ALIASES[alias.lower()] = name
    return entry


def unregister_architecture(name: str) -> None:
    entry = _ENTRIES.pop(name, None)
    if entry is not None:
        for alias in entry.aliases:
            _ALIASES.pop(alias.lower(), None)


def supported_architectures() -> list[str]:
    return sorted(set(_ENTRIES) | {k for k in _LAZY if k[0].isupper()})


def resolve_architecture(name: str) -> ArchitectureEntry:
    if name not in _ENTRIES and name.lower() not in _ALIASES:
        module = _LAZY.get(name) or _LAZY.get(name.lower())
        if module is not None:
            importlib.import_module(module)
    if name in _ENTRIES:
        return _ENTRIES[name]
    target = _ALIASES.get(name.lower())
    if target is not None:
        return _ENTRIES[target]
    raise ConfigError(
        f"unsupported architecture {name!r}; supported: {', '.join(supported_architectures())}"
    )


def config_from_dict(data: Mapping[str, Any], overrides: Mapping[str, Any] | None = None):
    """Parse a ``config.json`` body with the class its architecture registers."""
    merged = dict(data)
    if overrides:
        merged.update(overrides)
    entry = resolve_architecture(read_architecture(merged))
    return entry, entry.config_cls.from_dict(merged)
