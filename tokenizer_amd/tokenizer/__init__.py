"""Tokenizers, chosen by what a model folder's tokenizer.json declares.

`load_tokenizer(folder or file)` reads the file and hands it to the first registered kind that accepts it.  A kind
is registered with `register_tokenizer(name, accepts, build)`: `accepts(data) -> bool` looks at the parsed file
(its `model.type`, its pre-tokenizer), `build(data)` returns an object with `encode(text) -> ids`,
`decode_bytes(ids) -> bytes`, `decode(ids) -> str` and `vocab_size()`.  The byte-level BPE of the Qwen kind is the
one built in.
"""
from __future__ import annotations

import os
from typing import Callable

from .qwen_bpe import (Tokenizer, TokenizerError, UnknownToken, bytes_to_unicode_reverse, declares_byte_level_bpe,
                       read_tokenizer_json)

_KINDS: list[tuple[str, Callable[[dict], bool], Callable[[dict], object]]] = []


def register_tokenizer(name: str, accepts: Callable[[dict], bool], build: Callable[[dict], object],
                       replace: bool = False) -> None:
    known = [i for i, (kind, _, _) in enumerate(_KINDS) if kind == name]
    if known and not replace:
        raise ValueError(f"tokenizer kind {name!r} is already registered")
    for index in known:
        del _KINDS[index]
    _KINDS.append((name, accepts, build))


def registered_tokenizers() -> list[str]:
    return [name for name, _, _ in _KINDS]


def load_tokenizer(path: str):
    """The tokenizer of a model folder (its tokenizer.json) or of such a file, of the kind the file declares."""
    if os.path.isdir(path):
        path = os.path.join(path, "tokenizer.json")
    data = read_tokenizer_json(path)
    for _, accepts, build in _KINDS:
        if accepts(data):
            return build(data)
    model = data.get("model")
    declared = model.get("type") if isinstance(model, dict) else None
    raise TokenizerError(f"{path} declares a tokenizer (model type {declared!r}) that none of the registered kinds "
                         f"reads: {', '.join(registered_tokenizers())}")


register_tokenizer("byte_level_bpe", declares_byte_level_bpe, Tokenizer.from_json)

__all__ = ["Tokenizer", "TokenizerError", "UnknownToken", "bytes_to_unicode_reverse", "load_tokenizer",
           "register_tokenizer", "registered_tokenizers"]
