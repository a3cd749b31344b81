"""Streaming detokenizer for byte-level tokens (behaviour of qwen-infer/src/stream.rs:12-78).

A token may end in the middle of a UTF-8 character.  Complete text is handed out at once; an
incomplete tail waits for the next token; bytes that can never become a character turn into
one U+FFFD each time they are met; `finish` decodes whatever is left, lossily.
"""
from __future__ import annotations


class StreamDecoder:
    def __init__(self):
        self.pending = bytearray()

    def push(self, token_bytes: bytes) -> str:
        self.pending.extend(token_bytes)
        out = []
        while self.pending:
            try:
                out.append(self.pending.decode("utf-8"))
                self.pending.clear()
                break
            except UnicodeDecodeError as err:
                if err.start > 0:
                    out.append(self.pending[:err.start].decode("utf-8"))
                    del self.pending[:err.start]
                    continue
                # The error sits at the first byte: a truncated character waits, a wrong one is replaced.
                if err.reason == "unexpected end of data" and err.end == len(self.pending):
                    break
                out.append("�")
                del self.pending[:max(1, err.end - err.start)]
        return "".join(out)

    def finish(self) -> str:
        if not self.pending:
            return ""
        rest = self.pending.decode("utf-8", errors="replace")
        self.pending.clear()
        return rest
