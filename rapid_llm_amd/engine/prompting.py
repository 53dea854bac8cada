"""Chat prompts: the model folder's own template, or the prompt as it is.

The template is never in code.  It is read from the folder (``chat_template.jinja``, or the
``chat_template`` entry of ``tokenizer_config.json``) and rendered with the variables such
templates expect (``messages``, ``add_generation_prompt``, ``bos_token``, ``eos_token``), as
the reference renders it through its tokenizer (rapid_llm/utils/prompt_templates.py:19-57).
A folder without a template, or one that looks like a base checkpoint, gets its prompts
verbatim (:76-150): a name containing ``base`` is a base checkpoint; ``instruct``, ``chat`` or
``-it`` an instruction-tuned one; otherwise the architecture decides, through the flag its
registry entry carries (``register_architecture(..., chat_by_default=True)``): no
architecture is named here.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any

_INSTRUCT_HINTS = ("instruct", "chat", "-it")


def _special_token(entry: Any) -> str | None:
    """A special token of ``tokenizer_config.json``: a string, or a record with ``content``."""
    if isinstance(entry, str):
        return entry
    if isinstance(entry, dict) and isinstance(entry.get("content"), str):
        return entry["content"]
    return None


def read_tokenizer_config(model_dir: str | Path | None) -> dict:
    if model_dir is None:
        return {}
    path = Path(model_dir) / "tokenizer_config.json"
    if not path.is_file():
        return {}
    try:
        body = json.loads(path.read_text())
    except (OSError, json.JSONDecodeError):
        return {}
    return body if isinstance(body, dict) else {}


def read_chat_template(model_dir: str | Path) -> str | None:
    model_dir = Path(model_dir)
    path = model_dir / "chat_template.jinja"
    if path.is_file():
        return path.read_text()
    template = read_tokenizer_config(model_dir).get("chat_template")
    if isinstance(template, list):  # several named templates: the default one
        named = {t.get("name"): t.get("template") for t in template if isinstance(t, dict)}
        template = named.get("default")
    return template if isinstance(template, str) else None


def is_instruct(model_dir: str | Path) -> bool:
    name = Path(model_dir).name.lower()
    if "base" in name:
        return False
    if any(h in name for h in _INSTRUCT_HINTS):
        return True
    from ..config.registry import chat_by_default

    try:
        body = json.loads((Path(model_dir) / "config.json").read_text())
    except (OSError, json.JSONDecodeError):
        return False
    return isinstance(body, dict) and chat_by_default(body)


class ChatPrompter:
    """Formats conversations with one template."""

    def __init__(self, template: str, bos_token: str | None = None, eos_token: str | None = None) -> None:
        from datetime import datetime

        from jinja2.sandbox import ImmutableSandboxedEnvironment

        def raise_exception(message):
            raise ValueError(f"the chat template refused the conversation: {message}")

        def tojson(value, ensure_ascii=False, indent=None, separators=None, sort_keys=False):
            # the dialect's own filter: plain JSON text (jinja2's escapes <, >, & and quotes
            # for HTML, which would change the prompt's tokens)
            return json.dumps(value, ensure_ascii=ensure_ascii, indent=indent, separators=separators,
                              sort_keys=sort_keys)

        # what the templates of model folders may use beyond plain jinja2, as the tokenizer-side
        # rendering that the reference delegates to provides it
        # (rapid_llm/utils/prompt_templates.py:19-57): break / continue in loops, a tojson that
        # writes plain JSON, strftime_now and raise_exception
        env = ImmutableSandboxedEnvironment(
            trim_blocks=True, lstrip_blocks=True, extensions=["jinja2.ext.loopcontrols"]
        )
        env.filters["tojson"] = tojson
        env.globals["raise_exception"] = raise_exception
        env.globals["strftime_now"] = lambda fmt: datetime.now().strftime(fmt)
        self._template = env.from_string(template)
        self.bos_token = bos_token or ""
        self.eos_token = eos_token or ""

    def apply(self, messages: list[dict[str, str]], add_generation_prompt: bool = True) -> str:
        return self._template.render(
            messages=messages, add_generation_prompt=add_generation_prompt,
            bos_token=self.bos_token, eos_token=self.eos_token,
        )

    def insert_prompt(self, prompt: str) -> str:
        return self.apply([{"role": "user", "content": prompt}])


def build_prompter(model_dir: str | Path, use_template: bool = True) -> ChatPrompter | None:
    """The folder's prompter, or ``None``: prompts then go in as they are."""
    if not use_template or not is_instruct(model_dir):
        return None
    template = read_chat_template(model_dir)
    if template is None:
        return None
    cfg = read_tokenizer_config(model_dir)
    return ChatPrompter(template, _special_token(cfg.get("bos_token")), _special_token(cfg.get("eos_token")))
