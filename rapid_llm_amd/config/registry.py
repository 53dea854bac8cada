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
    # a checkpoint of this architecture whose folder name says neither "base" nor "instruct"
    # is a chat model and gets its folder's chat template (the reference keeps a list of such
    # model types beside its prompt code, rapid_llm/utils/prompt_templates.py:106-107)
    chat_by_default: bool = False


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
    chat_by_default: bool = False,
) -> ArchitectureEntry:
    if name in _ENTRIES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    entry = ArchitectureEntry(name, config_cls, build_spec, tuple(aliases), bool(chat_by_default))
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


def chat_by_default(config_body: Mapping[str, Any]) -> bool:
    """Whether the architecture a ``config.json`` body names registers its releases as chat
    models; ``False`` for a body that names none or one that is not registered."""
    try:
        return resolve_architecture(read_architecture(config_body)).chat_by_default
    except ConfigError:
        return False


def config_from_dict(data: Mapping[str, Any], overrides: Mapping[str, Any] | None = None):
    """Parse a ``config.json`` body with the class its architecture registers."""
    merged = dict(data)
    if overrides:
        merged.update(overrides)
    entry = resolve_architecture(read_architecture(merged))
    return entry, entry.config_cls.from_dict(merged)
