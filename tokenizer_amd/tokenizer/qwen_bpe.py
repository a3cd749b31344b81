"""Byte-level BPE read from a Hugging Face `tokenizer.json` of the Qwen kind.

What the file must look like is the reference's (src/qwen.rs:143-297): normalizer NFC; pre-tokenizer a
Sequence holding a Split step (its pattern a Regex, behaviour Isolated, not inverted) and a ByteLevel
step that brings no regex of its own; model BPE.  A vocabulary entry spells its bytes in the printable
alphabet of byte-level BPE (src/qwen.rs:96-121): every byte value must be a token; a merge ranks by its
place in the list and is looked up by the bytes it produces; added tokens are literals (`normalized:
false`), found in the text before anything else.

Encoding (src/rank.rs:368-447,536-586): cut the text at added tokens (leftmost first, the longest of
those that start at the same place), bring what lies between to NFC, cut that with the regex (what the
regex skips is a piece too), and inside every piece join the neighbouring pair of lowest rank (the
leftmost of equals) until no pair has a rank.
"""
from __future__ import annotations

import ctypes
import json
import unicodedata

import regex

from .. import host as _host


class TokenizerError(ValueError):
    pass


class UnknownToken(TokenizerError):
    def __init__(self, token: int):
        super().__init__(f"unknown token id {token}")
        self.token = token


def read_tokenizer_json(path: str) -> dict:
    try:
        with open(path, encoding="utf-8") as fh:
            data = json.load(fh)
    except OSError as err:
        raise TokenizerError(f"cannot read {path}: {err}") from None
    except json.JSONDecodeError as err:
        raise TokenizerError(f"{path} is not valid JSON: {err}") from None
    if not isinstance(data, dict):
        raise TokenizerError(f"{path} does not hold an object")
    return data


def declares_byte_level_bpe(data: dict) -> bool:
    """Whether a parsed tokenizer.json declares the kind this module reads: a BPE model behind a ByteLevel
    pre-tokenizer step (alone or in a Sequence)."""
    model, pre = data.get("model"), data.get("pre_tokenizer")
    if not isinstance(model, dict) or model.get("type") != "BPE" or not isinstance(pre, dict):
        return False
    steps = pre.get("pretokenizers") if pre.get("type") == "Sequence" else [pre]
    return any(isinstance(step, dict) and step.get("type") == "ByteLevel" for step in steps or [])


# ------------------------------------------------------------------------------------ the byte alphabet
_SELF_SPELLED = (range(0x21, 0x7F), range(0xA1, 0xAD), range(0xAE, 0x100))     # printable, kept as they are


def _byte_alphabet() -> list[str]:
    """The character that spells each byte value: printable Latin-1 bytes spell themselves, the other 68
    are numbered upwards from U+0100 in byte order."""
    spelled = [None] * 256
    for span in _SELF_SPELLED:
        for byte in span:
            spelled[byte] = chr(byte)
    following = 0x100
    for byte in range(256):
        if spelled[byte] is None:
            spelled[byte] = chr(following)
            following += 1
    return spelled


def bytes_to_unicode_reverse() -> dict[str, int]:
    """Character of a vocabulary string -> the byte it stands for."""
    return {ch: byte for byte, ch in enumerate(_byte_alphabet())}


# ------------------------------------------------------------------------------------- reading the file
class _Section:
    """One object of the file with a name for messages: `section["key"]` complains with the path to it."""

    def __init__(self, data, path: str):
        if not isinstance(data, dict):
            raise TokenizerError(f"{path} is missing or not an object")
        self.data, self.path = data, path

    def get(self, key: str, default=None):
        return self.data.get(key, default)

    def want(self, key: str, value, why: str = ""):
        found = self.data.get(key)
        if found != value:
            raise TokenizerError(f"{self.path}.{key} is {found!r} where {value!r} is needed" + (f" ({why})" if why else ""))

    def child(self, key: str) -> "_Section":
        return _Section(self.data.get(key), f"{self.path}.{key}")


class _TokenizerFile:
    """The parts of a parsed tokenizer.json that this tokenizer uses, each checked where it is read."""

    def __init__(self, data: dict):
        self.root = _Section(data, "tokenizer.json")
        self.alphabet = bytes_to_unicode_reverse()

    def check_normalizer(self) -> None:
        if not self.root.get("normalizer"):
            raise TokenizerError("tokenizer.json has no normalizer; texts are brought to NFC and the file must say so")
        self.root.child("normalizer").want("type", "NFC", "no other normalisation is applied")

    def split_regex(self) -> str:
        pre = self.root.child("pre_tokenizer")
        pre.want("type", "Sequence")
        steps = {}
        for index, step in enumerate(pre.get("pretokenizers") or []):
            section = _Section(step, f"{pre.path}.pretokenizers[{index}]")
            steps.setdefault(section.get("type"), section)
        for kind in ("Split", "ByteLevel"):
            if kind not in steps:
                raise TokenizerError(f"{pre.path} has no {kind} step")
        split, byte_level = steps["Split"], steps["ByteLevel"]
        split.want("behavior", "Isolated", "matches and the text between them are both kept as pieces")
        if split.get("invert"):
            raise TokenizerError(f"{split.path}.invert is set; an inverted split is not handled")
        pattern = split.child("pattern").get("Regex")
        if not isinstance(pattern, str):
            raise TokenizerError(f"{split.path}.pattern holds no Regex")
        if byte_level.get("use_regex"):
            raise TokenizerError(f"{byte_level.path}.use_regex is set; pieces are cut by the Split step's regex alone")
        return pattern

    def spell(self, text: str, what: str) -> bytes:
        try:
            return bytes(self.alphabet[ch] for ch in text)
        except KeyError as stray:
            raise TokenizerError(f"{what} {text!r} holds U+{ord(stray.args[0]):04X}, which spells no byte") from None

    def byte_vocab(self) -> dict[bytes, int]:
        model = self.root.child("model")
        model.want("type", "BPE")
        ids: dict[bytes, int] = {}
        for text, token in (model.get("vocab") or {}).items():
            raw = self.spell(text, "vocabulary entry")
            if raw in ids:
                raise TokenizerError(f"vocabulary ids {ids[raw]} and {token} spell the same bytes")
            ids[raw] = token
        absent = [byte for byte in range(256) if bytes([byte]) not in ids]
        if absent:
            raise TokenizerError(f"missing single-byte token {absent[0]}"
                                 + (f" (and {len(absent) - 1} more)" if len(absent) > 1 else ""))
        return ids

    def merge_ranks(self, ids: dict[bytes, int]) -> dict[bytes, int]:
        ranks: dict[bytes, int] = {}
        for rank, entry in enumerate(self.root.child("model").get("merges") or []):
            halves = entry.split(" ") if isinstance(entry, str) else list(entry)
            if len(halves) == 1:
                raise TokenizerError(f"merge {rank} ({entry!r}) has no space between its halves")
            if len(halves) != 2 or not all(halves):
                raise TokenizerError(f"merge {rank} ({entry!r}) is not a pair")
            left, right = (self.spell(half, f"merge {rank}:") for half in halves)
            for side in (left, right, left + right):
                if side not in ids:
                    raise TokenizerError(f"merge {rank} ({entry!r}): {side!r} is not in the vocab")
            if left + right in ranks:
                raise TokenizerError(f"merges {ranks[left + right]} and {rank} produce the same bytes")
            ranks[left + right] = rank
        return ranks

    def literals(self) -> dict[str, int]:
        found: dict[str, int] = {}
        for index, entry in enumerate(self.root.get("added_tokens") or []):
            item = _Section(entry, f"tokenizer.json.added_tokens[{index}]")
            content, token = item.get("content"), item.get("id")
            if not content or not isinstance(token, int):
                raise TokenizerError(f"{item.path} needs a content that is not empty and an id")
            if item.get("normalized", True):
                raise TokenizerError(f"{item.path} ({content!r}) is normalized; added tokens are matched as literals only")
            if content in found:
                raise TokenizerError(f"{item.path} ({content!r}) is listed twice")
            found[content] = token
        return found


class _MergeCore:
    """The merges inside a piece and the way back from ids to bytes, in the host library (csrc/host/bpe_core.cpp)."""

    def __init__(self, encoder: dict[bytes, int], ranks: dict[bytes, int], specials: dict[str, int]):
        self._lib = _host.lib()
        self._core = self._lib.ta_bpe_new()
        for raw, token in encoder.items():
            if self._lib.ta_bpe_add_token(self._core, token, raw, len(raw), 1) != 0:
                raise TokenizerError(f"token id {token} or its bytes {raw!r} are taken already")
        for text, token in specials.items():
            raw = text.encode("utf-8")
            if self._lib.ta_bpe_add_token(self._core, token, raw, len(raw), 0) != 0:
                raise TokenizerError(f"token id {token} of {text!r} is taken already")
        for merged, rank in ranks.items():
            self._lib.ta_bpe_add_merge(self._core, merged, len(merged), rank)
        self._ids = (ctypes.c_int32 * 256)()

    def __del__(self):
        if getattr(self, "_core", None):
            self._lib.ta_bpe_delete(self._core)
            self._core = None

    def piece(self, piece: bytes, ids: list[int]) -> None:
        count = self._lib.ta_bpe_encode_piece(self._core, piece, len(piece), self._ids, len(self._ids))
        if count < 0 and count > -(1 << 31):                 # the piece has more parts than the buffer holds
            self._ids = (ctypes.c_int32 * (-count))()
            count = self._lib.ta_bpe_encode_piece(self._core, piece, len(piece), self._ids, len(self._ids))
        if count < 0:
            raise TokenizerError(f"piece {piece!r} does not break down into tokens of the vocabulary")
        ids.extend(self._ids[:count])

    def bytes_of(self, ids) -> bytes:
        tokens = [int(t) for t in ids]
        if any(not -(1 << 31) <= t < (1 << 31) for t in tokens):
            raise UnknownToken(next(t for t in tokens if not -(1 << 31) <= t < (1 << 31)))
        array = (ctypes.c_int32 * max(1, len(tokens)))(*tokens)
        bad = ctypes.c_int32(0)
        out = ctypes.create_string_buffer(max(1, 8 * len(tokens)))
        size = self._lib.ta_bpe_decode(self._core, array, len(tokens), out, len(out), ctypes.byref(bad))
        if size < 0 and size > -(1 << 31):
            out = ctypes.create_string_buffer(-size)
            size = self._lib.ta_bpe_decode(self._core, array, len(tokens), out, len(out), ctypes.byref(bad))
        if size < 0:
            raise UnknownToken(tokens[bad.value])
        return out.raw[:size]


class Tokenizer:
    def __init__(self, encoder, decoder, ranks, specials, pattern: str):
        self.encoder: dict[bytes, int] = encoder
        self.decoder: list[bytes | None] = decoder
        self.ranks: dict[bytes, int] = ranks
        self.specials: dict[str, int] = specials
        self._core = _MergeCore(encoder, ranks, specials)
        try:
            self.pattern = regex.compile(pattern)
        except regex.error as err:
            raise TokenizerError(f"split pattern does not compile: {err}") from None
        # Leftmost match, and among literals that start there the longest: the alternatives are tried in order.
        by_length = sorted(specials, key=len, reverse=True)
        self._literal = regex.compile("|".join(regex.escape(text) for text in by_length)) if specials else None

    # -------------------------------------------------------------------- loading
    @classmethod
    def load_qwen(cls, path: str) -> "Tokenizer":
        return cls.from_json(read_tokenizer_json(path))

    @staticmethod
    def load(path: str):
        """The tokenizer of a model folder or tokenizer.json, of whichever registered kind the file declares."""
        from . import load_tokenizer
        return load_tokenizer(path)

    @classmethod
    def from_json(cls, data: dict) -> "Tokenizer":
        source = _TokenizerFile(data)
        source.check_normalizer()
        pattern = source.split_regex()
        ids = source.byte_vocab()
        ranks = source.merge_ranks(ids)
        literals = source.literals()
        # id -> bytes for both kinds of token; no id may mean two things.
        table: dict[int, bytes] = {}
        for raw, token in list(ids.items()) + [(text.encode("utf-8"), token) for text, token in literals.items()]:
            if token in table:
                raise TokenizerError(f"token id {token} is given to {table[token]!r} and to {raw!r}")
            table[token] = raw
        decoder: list[bytes | None] = [None] * (max(table) + 1)
        for token, raw in table.items():
            if token < 0:
                raise TokenizerError(f"token id {token} is negative")
            decoder[token] = raw
        return cls(ids, decoder, ranks, literals, pattern)

    # ------------------------------------------------------------------- encoding
    def vocab_size(self) -> int:
        return len(self.decoder)

    def encode(self, text: str) -> list[int]:
        ids: list[int] = []
        at = 0
        if self._literal is not None:
            for match in self._literal.finditer(text):
                self._encode_ordinary(text[at:match.start()], ids)
                ids.append(self.specials[match.group()])
                at = match.end()
        self._encode_ordinary(text[at:], ids)
        return ids

    def _encode_ordinary(self, text: str, ids: list[int]) -> None:
        if not text:
            return
        text = unicodedata.normalize("NFC", text)
        at = 0
        for match in self.pattern.finditer(text):
            if match.end() == match.start():
                continue
            if match.start() > at:
                self._encode_piece(text[at:match.start()].encode("utf-8"), ids)    # what the regex skipped
            self._encode_piece(match.group().encode("utf-8"), ids)
            at = match.end()
        if at < len(text):
            self._encode_piece(text[at:].encode("utf-8"), ids)

    def _encode_piece(self, piece: bytes, ids: list[int]) -> None:
        self._core.piece(piece, ids)

    # ------------------------------------------------------------------- decoding
    def decode_bytes(self, ids) -> bytes:
        return self._core.bytes_of(ids)

    def decode(self, ids) -> str:
        return self.decode_bytes(ids).decode("utf-8", errors="replace")
