"""Byte-level BPE read from a Hugging Face `tokenizer.json` of the Qwen kind.

Loader rules follow src/qwen.rs:143-297 of the reference: the normalizer must be NFC; the
pre-tokenizer a Sequence with a Split step (a Regex, behaviour Isolated, not inverted) and a
ByteLevel step without its own regex; the model BPE.  Vocabulary strings are mapped back to
bytes through the inverse of GPT-2's `bytes_to_unicode` (src/qwen.rs:96-121); all 256 single
bytes must be tokens; a merge's rank is its index in the list; added tokens must be
`normalized: false` and are matched literally before anything else.

Encoding follows src/rank.rs:368-447,536-586: split out the earliest added token (the longest
on a tie), NFC the text between, split it with the regex keeping unmatched gaps as pieces,
and in every piece merge the adjacent pair of lowest rank (leftmost on a tie) until none is left.
"""
from __future__ import annotations

import json
import unicodedata

import regex


class TokenizerError(ValueError):
    pass


class UnknownToken(TokenizerError):
    def __init__(self, token: int):
        super().__init__(f"unknown token id {token}")
        self.token = token


def bytes_to_unicode_reverse() -> dict[str, int]:
    """Character of a vocabulary string -> the byte it stands for."""
    keep = list(range(ord("!"), ord("~") + 1)) + list(range(0xA1, 0xAD)) + list(range(0xAE, 0x100))
    codes = list(keep)
    extra = 0
    for byte in range(256):
        if byte not in keep:
            keep.append(byte)
            codes.append(256 + extra)
            extra += 1
    return {chr(code): byte for byte, code in zip(keep, codes)}


class Tokenizer:
    def __init__(self, encoder, decoder, ranks, specials, pattern: str):
        self.encoder: dict[bytes, int] = encoder
        self.decoder: list[bytes | None] = decoder
        self.ranks: dict[bytes, int] = ranks
        self.specials: dict[str, int] = specials
        try:
            self.pattern = regex.compile(pattern)
        except regex.error as err:
            raise TokenizerError(f"split pattern does not compile: {err}") from None

    # -------------------------------------------------------------------- loading
    @classmethod
    def load_qwen(cls, path: str) -> "Tokenizer":
        try:
            with open(path, encoding="utf-8") as fh:
                data = json.load(fh)
        except OSError as err:
            raise TokenizerError(f"cannot read {path}: {err}") from None
        except json.JSONDecodeError as err:
            raise TokenizerError(f"{path} is not valid JSON: {err}") from None
        return cls.from_json(data)

    @classmethod
    def from_json(cls, data: dict) -> "Tokenizer":
        normalizer = data.get("normalizer")
        if not normalizer:
            raise TokenizerError("tokenizer.json has no normalizer")
        if normalizer.get("type") != "NFC":
            raise TokenizerError(f"expected an NFC normalizer, found {normalizer.get('type')}")
        pre = data.get("pre_tokenizer") or {}
        if pre.get("type") != "Sequence":
            raise TokenizerError(f"expected a Sequence pre-tokenizer, found {pre.get('type')}")
        pattern = cls._split_pattern(pre)
        model = data.get("model") or {}
        if model.get("type") != "BPE":
            raise TokenizerError(f"expected a BPE model, found {model.get('type')}")
        reverse = bytes_to_unicode_reverse()

        def unmap(token: str) -> bytes:
            try:
                return bytes(reverse[ch] for ch in token)
            except KeyError as err:
                raise TokenizerError(f"vocab char U+{ord(err.args[0]):04X} is not a bytes_to_unicode scalar") from None

        encoder: dict[bytes, int] = {}
        max_id = 0
        for token, token_id in model.get("vocab", {}).items():
            raw = unmap(token)
            if raw in encoder:
                raise TokenizerError(f"duplicate vocab bytes for id {token_id}")
            encoder[raw] = token_id
            max_id = max(max_id, token_id)
        for byte in range(256):
            if bytes([byte]) not in encoder:
                raise TokenizerError(f"missing single-byte token {byte}")
        ranks: dict[bytes, int] = {}
        for index, merge in enumerate(model.get("merges", [])):
            if isinstance(merge, list):
                merge = " ".join(merge)
            left, sep, right = merge.partition(" ")
            if not sep:
                raise TokenizerError(f"merge {index} has no space")
            if not left or not right or " " in right:
                raise TokenizerError(f"merge {index} is not two bytes_to_unicode tokens")
            left_b, right_b = unmap(left), unmap(right)
            if left_b not in encoder or right_b not in encoder:
                raise TokenizerError(f"merge {index} names a token that is not in the vocab")
            merged = left_b + right_b
            if merged not in encoder:
                raise TokenizerError(f"merge {index} concatenation is not in the vocab")
            if merged in ranks:
                raise TokenizerError(f"merge {index} repeats a byte string")
            ranks[merged] = index
        added = data.get("added_tokens", [])
        for item in added:
            max_id = max(max_id, item["id"])
        decoder: list[bytes | None] = [None] * (max_id + 1)
        for raw, token_id in encoder.items():
            if decoder[token_id] is not None:
                raise TokenizerError(f"duplicate token id {token_id}")
            decoder[token_id] = raw
        specials: dict[str, int] = {}
        for item in added:
            if item.get("normalized", True):
                raise TokenizerError(f"added token {item['content']!r} is normalized; only normalized=false is supported")
            if not item["content"]:
                raise TokenizerError("added token content is empty")
            if decoder[item["id"]] is not None:
                raise TokenizerError(f"added token id {item['id']} already belongs to a vocab token")
            decoder[item["id"]] = item["content"].encode("utf-8")
            if item["content"] in specials:
                raise TokenizerError(f"duplicate added token {item['content']!r}")
            specials[item["content"]] = item["id"]
        return cls(encoder, decoder, ranks, specials, pattern)

    @staticmethod
    def _split_pattern(pre: dict) -> str:
        steps = pre.get("pretokenizers", [])
        split = next((s for s in steps if s.get("type") == "Split"), None)
        if split is None:
            raise TokenizerError("pre-tokenizer has no Split step")
        if split.get("behavior") != "Isolated":
            raise TokenizerError(f"expected Split behavior Isolated, found {split.get('behavior')!r}")
        if split.get("invert", False):
            raise TokenizerError("Split invert=true is not supported")
        pattern = (split.get("pattern") or {}).get("Regex")
        if pattern is None:
            raise TokenizerError("Split step has no Regex pattern")
        byte_level = next((s for s in steps if s.get("type") == "ByteLevel"), None)
        if byte_level is None:
            raise TokenizerError("pre-tokenizer has no ByteLevel step")
        if byte_level.get("use_regex", False):
            raise TokenizerError("ByteLevel use_regex must be false; the Split step owns the regex")
        return pattern

    # ------------------------------------------------------------------- encoding
    def vocab_size(self) -> int:
        return len(self.decoder)

    def encode(self, text: str) -> list[int]:
        ids: list[int] = []
        rest = text
        while True:
            found = self._earliest_special(rest)
            if found is None:
                self._push_ordinary(rest, ids)
                return ids
            start, token = found
            self._push_ordinary(rest[:start], ids)
            ids.append(self.specials[token])
            rest = rest[start + len(token):]

    def _earliest_special(self, text: str):
        best = None
        for token in self.specials:
            at = text.find(token)
            if at < 0:
                continue
            if best is None or at < best[0] or (at == best[0] and len(token) > len(best[1])):
                best = (at, token)
        return best

    def _push_ordinary(self, text: str, ids: list[int]) -> None:
        if not text:
            return
        text = unicodedata.normalize("NFC", text)
        at = 0
        for match in self.pattern.finditer(text):
            if match.start() > at:
                self._push_piece(text[at:match.start()].encode("utf-8"), ids)   # a gap is a piece too
            if match.end() > match.start():
                self._push_piece(match.group().encode("utf-8"), ids)
            at = max(at, match.end())
        if at < len(text):
            self._push_piece(text[at:].encode("utf-8"), ids)

    def _push_piece(self, piece: bytes, ids: list[int]) -> None:
        if not piece:
            return
        parts = [piece[i:i + 1] for i in range(len(piece))]
        while len(parts) > 1:
            best_rank, best_at = None, -1
            for i in range(len(parts) - 1):
                rank = self.ranks.get(parts[i] + parts[i + 1])
                if rank is not None and (best_rank is None or rank < best_rank):
                    best_rank, best_at = rank, i
            if best_rank is None:
                break
            parts[best_at:best_at + 2] = [parts[best_at] + parts[best_at + 1]]
        ids.extend(self.encoder[part] for part in parts)

    # ------------------------------------------------------------------- decoding
    def decode_bytes(self, ids) -> bytes:
        out = bytearray()
        for token in ids:
            raw = self.decoder[token] if 0 <= token < len(self.decoder) else None
            if raw is None:
                raise UnknownToken(token)
            out.extend(raw)
        return bytes(out)

    def decode(self, ids) -> str:
        return self.decode_bytes(ids).decode("utf-8", errors="replace")
