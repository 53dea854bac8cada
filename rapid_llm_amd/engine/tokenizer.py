"""Text in and out: a ``tokenizer.json`` read with the ``tokenizers`` package, if the model
folder has one.  A folder of random weights has none; prompts are then lists of token ids
and completions come back as ids."""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any


class TextTokenizer:
    def __init__(self, path: str | Path) -> None:
        from tokenizers import Tokenizer

        self._tok = Tokenizer.from_file(str(path))

    def encode(self, text: str) -> list[int]:
        return list(self._tok.encode(text, add_special_tokens=False).ids)

    def decode(self, ids, skip_special_tokens: bool = True) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=skip_special_tokens)

    def token_to_id(self, token: str) -> int | None:
        return self._tok.token_to_id(token)


def load_tokenizer(model_dir: str | Path) -> TextTokenizer | None:
    path = Path(model_dir) / "tokenizer.json"
    return TextTokenizer(path) if path.is_file() else None


def tokenizer_eos_token_id(model_dir: str | Path | None, tokenizer: Any = None) -> int | None:
    """The tokenizer's own end-of-sequence id: ``eos_token_id`` of the tokenizer object if it
    has one, else ``eos_token`` of ``tokenizer_config.json`` (a string or a record with
    ``content``) looked up in the vocabulary."""
    eos_id = getattr(tokenizer, "eos_token_id", None)
    if isinstance(eos_id, int):
        return eos_id
    from .prompting import _special_token, read_tokenizer_config

    cfg = read_tokenizer_config(model_dir)
    if isinstance(cfg.get("eos_token_id"), int):
        return int(cfg["eos_token_id"])
    token = _special_token(cfg.get("eos_token"))
    if token is not None and tokenizer is not None and hasattr(tokenizer, "token_to_id"):
        found = tokenizer.token_to_id(token)
        if found is not None:
            return int(found)
    return None


def load_stop_token_ids(model_dir: str | Path | None, config_eos=(), tokenizer: Any = None) -> set[int]:
    """The tokenizer's end-of-sequence id *and* ``eos_token_id`` of ``generation_config.json``
    (an int or a list) and of ``config.json`` (rapid_llm/engine/stop_criteria.py:29-54: an
    instruction-tuned model usually ends on another token than the tokenizer's default, so
    both count)."""
    stop = {int(t) for t in config_eos}
    own = tokenizer_eos_token_id(model_dir, tokenizer)
    if own is not None:
        stop.add(own)
    if model_dir is not None:
        path = Path(model_dir) / "generation_config.json"
        if path.is_file():
            try:
                eos = json.loads(path.read_text()).get("eos_token_id")
            except json.JSONDecodeError:
                eos = None
            if isinstance(eos, int):
                stop.add(eos)
            elif isinstance(eos, list):
                stop.update(int(t) for t in eos)
    return stop


class Detokenizer:
    """Incremental decoding: text is released only once it no longer ends in an incomplete
    character (a multi-byte character may span tokens)."""

    def __init__(self, tokenizer: Any) -> None:
        self.tokenizer = tokenizer
        self.ids: list[int] = []
        self.prefix = 0  # ids[prefix:read] is context already released
        self.read = 0

    def append(self, token: int) -> str:
        self.ids.append(token)
        before = self.tokenizer.decode(self.ids[self.prefix : self.read])
        now = self.tokenizer.decode(self.ids[self.prefix :])
        if len(now) > len(before) and not now.endswith("�"):
            self.prefix = self.read
            self.read = len(self.ids)
            return now[len(before) :]
        return ""
