"""Generation parameters, the per-sequence sampling state machine and the stop-string hold.

Names and meanings follow qwen-infer/src/generate.rs: `GenerateParams` (45-73), `Generated`
(76-101), `StopReason` (17-33), `Control` (36-42), `SampleCursor` (172-338), `StopHold`
(433-501).  The cursor owns one sequence's random generator, decoded text and stop-string
hold; the caller runs the model and hands logits (or an id already picked on the device) back.
"""
from __future__ import annotations

import dataclasses
import enum
from typing import Callable

from ..sampling.host import Rng, SampleError, check_params, sample_with_uniform, greedy_token
from .stream import StreamDecoder


class StopReason(enum.Enum):
    MaxTokens = "MaxTokens"     # max_tokens ids were sampled, none was an EOS id
    Eos = "Eos"                 # the sampled id is in `eos`; it is neither stored nor decoded
    StopString = "StopString"   # a stop string occurred in the decoded text; it is never emitted
    Cancelled = "Cancelled"     # the chunk callback returned Control.Stop


class Control(enum.Enum):
    Continue = "Continue"
    Stop = "Stop"


@dataclasses.dataclass
class GenerateParams:
    max_tokens: int = 20
    temperature: float = 0.0    # 0 is greedy
    top_p: float = 1.0
    seed: int = 0
    eos: list[int] = dataclasses.field(default_factory=list)
    stop: list[str] = dataclasses.field(default_factory=list)

    @classmethod
    def greedy(cls, max_tokens: int) -> "GenerateParams":
        return cls(max_tokens=max_tokens, temperature=0.0, top_p=1.0, seed=0, eos=[], stop=[])


@dataclasses.dataclass
class Sampled:
    tokens: list[int]
    text: str
    chunks: list[str]
    reason: StopReason
    completion_tokens: int


@dataclasses.dataclass
class Generated:
    tokens: list[int]           # sampled ids without an EOS id; a stop-string token is included
    text: str                   # decoded text with stop strings removed
    chunks: list[str]           # pieces as they became safe to show; joined they are `text`
    reason: StopReason
    completion_tokens: int      # ids the model sampled, counting an EOS id
    prefill: float = 0.0        # seconds of the prompt's forward
    decode: float = 0.0         # seconds of the decode forwards (sampling included)


def validate(params: GenerateParams) -> None:
    """generate.rs:409-426."""
    check_params(params.temperature, params.top_p)
    if params.max_tokens < 0:
        raise SampleError("max_tokens is negative")
    if any(stop == "" for stop in params.stop):
        raise SampleError("stop strings must be non-empty")


class StopHold:
    """Decoded text on its way out, with stop strings watched for (behaviour of generate.rs:433-501).

    Only the text that has not been handed out yet is kept: the `tail`.  After every push it is the longest end
    of the text that could still be the beginning of a stop string, and nothing else; so a stop string, which
    never starts inside text that was let go, is always found inside tail + new chunk, and a push costs what
    the chunk and the stop strings are long, however much text went before.  A completed stop string ends the
    stream: the text before it goes out, the stop string itself and what follows never do.
    """

    def __init__(self):
        self.tail = ""
        self.handed_out = 0          # characters given to the caller so far
        self.stopped = False

    @staticmethod
    def _first_stop(window: str, stops: list[str]) -> int:
        """Where the earliest stop string starts in `window`, or -1."""
        starts = [at for at in (window.find(stop) for stop in stops) if at >= 0]
        return min(starts) if starts else -1

    @staticmethod
    def _open_end(window: str, stops: list[str]) -> int:
        """How many characters at the end of `window` begin a stop string without completing it."""
        longest = 0
        for stop in stops:
            for size in range(min(len(window), len(stop) - 1), longest, -1):
                if window.endswith(stop[:size]):
                    longest = size
                    break
        return longest

    def push(self, chunk: str, stops: list[str]) -> tuple[bool, str]:
        """Returns (a stop string was completed, text that may go out now)."""
        if self.stopped:
            return True, ""
        window = self.tail + chunk
        cut = self._first_stop(window, stops) if stops else -1
        if cut >= 0:
            self.stopped, self.tail = True, ""
            self.handed_out += cut
            return True, window[:cut]
        keep = self._open_end(window, stops) if stops else 0
        out = window[:len(window) - keep]
        self.tail = window[len(window) - keep:]
        self.handed_out += len(out)
        return False, out

    def finish(self) -> str:
        """What was held back in case it grew into a stop string, now that nothing more comes."""
        out, self.tail = self.tail, ""
        self.handed_out += len(out)
        return out


TokenBytes = Callable[[int], bytes]
OnChunk = Callable[[str], Control]


def _no_bytes(_id: int) -> bytes:
    return b""


def _go_on(_piece: str) -> Control:
    return Control.Continue


class SampleCursor:
    """One sequence's sampler.  `push_logits` draws from logits on the host; `push_token` takes an id
    that the device already picked with this cursor's parameters (and, for a warm draw, the uniform
    number from `next_uniform`).  Both return the id to forward next, or a finished `Sampled`."""

    def __init__(self, params: GenerateParams):
        validate(params)
        self.params = params
        self.rng = Rng(params.seed)
        self.decoder = StreamDecoder()
        self.held = StopHold()
        self.tokens: list[int] = []
        self.chunks: list[str] = []
        self.text = ""
        self.produced = 0

    # ------------------------------------------------------------------- drawing
    @property
    def exhausted(self) -> bool:
        return self.produced >= self.params.max_tokens

    @property
    def is_greedy(self) -> bool:
        return self.params.temperature == 0

    def next_uniform(self) -> float:
        """The uniform number of the next warm draw (consumes it)."""
        return self.rng.random_f32()

    def push_logits(self, logits, token_bytes: TokenBytes = _no_bytes, on_chunk: OnChunk = _go_on):
        if self.exhausted:
            return self.finish(StopReason.MaxTokens, on_chunk)
        if self.is_greedy:
            token = greedy_token(logits)
        else:
            token = sample_with_uniform(logits, self.params.temperature, self.params.top_p, self.next_uniform())
        return self.push_token(token, token_bytes, on_chunk)

    def push_token(self, token: int, token_bytes: TokenBytes = _no_bytes, on_chunk: OnChunk = _go_on):
        """generate.rs:232-284 after the draw."""
        if self.exhausted:
            return self.finish(StopReason.MaxTokens, on_chunk)
        token = int(token)
        if token in self.params.eos:
            self.produced += 1
            return self.finish(StopReason.Eos, on_chunk)
        piece = self.decoder.push(token_bytes(token))
        stopped, chunk = self.held.push(piece, self.params.stop)
        self.tokens.append(token)
        self.produced += 1
        control = self._observe(on_chunk, chunk)
        if stopped:
            return self.snapshot(StopReason.Cancelled if control == Control.Stop else StopReason.StopString)
        if control == Control.Stop:
            return self.snapshot(StopReason.Cancelled)
        if self.exhausted:
            return self.finish(StopReason.MaxTokens, on_chunk)
        return token

    def finish_without_sample(self, on_chunk: OnChunk = _go_on) -> Sampled:
        """`max_tokens == 0`: the prompt was still run, nothing is drawn (generate.rs:286-291)."""
        return self.finish(StopReason.MaxTokens, on_chunk)

    # ------------------------------------------------------------------ finishing
    def snapshot(self, reason: StopReason) -> Sampled:
        return Sampled(list(self.tokens), self.text, list(self.chunks), reason, self.produced)

    def finish(self, reason: StopReason, on_chunk: OnChunk = _go_on) -> Sampled:
        """Flush the decoder's tail and the held-back text for MaxTokens and Eos (generate.rs:303-337)."""
        if reason in (StopReason.MaxTokens, StopReason.Eos):
            flushed = self.decoder.finish()
            if flushed:
                stopped, chunk = self.held.push(flushed, self.params.stop)
                if stopped:
                    control = self._observe(on_chunk, chunk)
                    reason = StopReason.Cancelled if control == Control.Stop else StopReason.StopString
                else:
                    first = self._observe(on_chunk, chunk)
                    second = self._observe(on_chunk, self.held.finish())
                    if Control.Stop in (first, second):
                        reason = StopReason.Cancelled
            elif self._observe(on_chunk, self.held.finish()) == Control.Stop:
                reason = StopReason.Cancelled
        return self.snapshot(reason)

    def _observe(self, on_chunk: OnChunk, piece: str) -> Control:
        if piece:
            self.chunks.append(piece)
            self.text += piece
        return on_chunk(piece) or Control.Continue


def parse_eos_token_ids(text: str) -> list[int]:
    """`eos_token_id` of a generation_config.json: one integer or a non-empty list
    (qwen-infer/src/lib.rs:84-107)."""
    import json
    value = json.loads(text)
    if not isinstance(value, dict) or "eos_token_id" not in value:
        raise ValueError("generation config has no eos_token_id")
    eos = value["eos_token_id"]
    if isinstance(eos, int) and not isinstance(eos, bool):
        ids = [eos]
    elif isinstance(eos, list):
        if not eos:
            raise ValueError("eos_token_id is empty")
        if any(isinstance(item, bool) or not isinstance(item, int) for item in eos):
            raise ValueError("eos_token_id entry is not an integer")
        ids = list(eos)
    else:
        raise ValueError("eos_token_id is not an integer or a list")
    if any(not 0 <= item < (1 << 32) for item in ids):
        raise ValueError("eos id does not fit in u32")
    return ids


def load_eos_token_ids(path: str) -> list[int]:
    with open(path) as fh:
        return parse_eos_token_ids(fh.read())
