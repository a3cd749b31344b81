"""Continuous-batching scheduler above the step function.

Policy follows qwen-server/src/engine.rs: a FIFO of waiting requests and a running batch;
admission looks at the front of the queue only and reserves pages for the whole prompt
(458-517); each iteration grows the running sequences oldest first and, when pages run out,
preempts the newest sequence, which gives back everything and is recomputed later (561-668);
preempted sequences return to the front of the queue, oldest first (369-376); a sequence that
cannot fit in the whole pool fails with a message (473-487, 670-685).

Beyond the reference, one iteration is a single mixed batch under a token budget: one token
for every decoding sequence first, then portions of prompts in order of arrival.  A preempted
sequence is recomputed from its prompt and the tokens it sampled so far, and nothing is
sampled again for positions that already have a token.
"""
from __future__ import annotations

import collections
import dataclasses
import time
from typing import Callable

from ..cache.allocator import pages_for_len
from .batch import StepEntry
from .generate import (Control, GenerateParams, Generated, SampleCursor, Sampled, StopReason, _go_on,
                       _no_bytes)


@dataclasses.dataclass
class SchedulerConfig:
    """`max_batch_size`, `max_waiting`, `num_blocks` and `prefix_cache` carry the names and defaults of
    qwen-server/src/lib.rs:33-56; the token budget and the portion size are this engine's."""
    max_batch_size: int = 8
    max_waiting: int = 32
    num_blocks: int = 256
    prefix_cache: bool = True
    max_num_batched_tokens: int = 2048
    prefill_chunk: int | None = None


@dataclasses.dataclass
class EngineStats:
    """Counters of qwen-server/src/engine.rs:64-86 that make sense without a server."""
    requests_finished: int = 0
    requests_failed: int = 0
    max_running: int = 0
    preemptions: int = 0
    last_preempted_id: int = 0
    peak_blocks: int = 0
    peak_occupied: int = 0
    steps: int = 0
    tokens_forwarded: int = 0


class QueueFull(RuntimeError):
    pass


@dataclasses.dataclass
class Failure:
    message: str


class Sequence:
    def __init__(self, seq_id: int, prompt: list[int], params: GenerateParams, token_bytes, on_chunk):
        self.id = seq_id
        self.prompt = list(prompt)
        self.tokens = list(prompt)       # prompt and every sampled id that is to be forwarded
        self.params = params
        self.cursor = SampleCursor(params)
        self.token_bytes = token_bytes
        self.on_chunk = on_chunk
        self.computed = 0                # tokens whose keys and values are in the cache
        self.prefill = 0.0
        self.decode = 0.0
        self.result: Generated | Failure | None = None

    @property
    def sampled(self) -> int:
        return len(self.tokens) - len(self.prompt)

    @property
    def remaining(self) -> int:
        return len(self.tokens) - self.computed

    @property
    def decoding(self) -> bool:
        return self.sampled > 0 and self.remaining == 1


class Scheduler:
    """Admits requests, cuts prompts into portions, decodes, finishes and frees.

    `engine` needs: `.cache` (a CacheManager), `.step(entries) -> logits`, `.argmax(logits, rows) ->
    list[int]`, `.max_positions`, and for warm requests `.sample(logits, rows, temperature, top_p, uniform)
    -> list[int]` or, without it, `.rows_to_host(logits, rows) -> float32 array` (drawn on the host then).
    """

    def __init__(self, engine, config: SchedulerConfig | None = None):
        self.engine = engine
        self.cache = engine.cache
        self.config = config or SchedulerConfig()
        self.waiting: collections.deque[Sequence] = collections.deque()
        self.running: list[Sequence] = []
        self.finished: dict[int, Generated | Failure] = {}
        self.stats = EngineStats()
        self._next_id = 1

    # ------------------------------------------------------------------- requests
    def add_request(self, prompt: list[int], params: GenerateParams | None = None,
                    token_bytes: Callable[[int], bytes] = _no_bytes,
                    on_chunk: Callable[[str], Control] = _go_on) -> int:
        """Queue a request; returns its id.  Problems with the request itself are recorded as a failed
        result under that id (as the reference answers them on the request's own channel)."""
        params = params or GenerateParams()
        if len(self.waiting) >= self.config.max_waiting:
            raise QueueFull(f"{len(self.waiting)} requests are already waiting")
        seq_id = self._next_id
        self._next_id += 1
        if not prompt:
            self._fail_new(seq_id, "prompt encoded to no tokens")          # engine.rs:414-423
            return seq_id
        limit = self.engine.max_positions
        if len(prompt) + params.max_tokens > limit:                        # http.rs:259-275
            self._fail_new(seq_id, f"prompt of {len(prompt)} tokens plus max_tokens {params.max_tokens} "
                                   f"exceeds max_position_embeddings {limit}")
            return seq_id
        try:
            seq = Sequence(seq_id, prompt, params, token_bytes, on_chunk)
        except ValueError as err:
            self._fail_new(seq_id, str(err))
            return seq_id
        self.waiting.append(seq)
        return seq_id

    def _fail_new(self, seq_id: int, message: str) -> None:
        self.finished[seq_id] = Failure(message)
        self.stats.requests_failed += 1

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ admission
    def _pages_to_admit(self, seq: Sequence) -> int:
        # A new request needs its prompt; one that already sampled also gets room for the next token, so
        # that it is not evicted again at once (engine.rs:696-704).
        length = len(seq.tokens) + (1 if seq.sampled else 0)
        return pages_for_len(length, self.cache.page_size)

    def _admit(self) -> None:
        while self.waiting and len(self.running) < self.config.max_batch_size:
            seq = self.waiting[0]
            needed = self._pages_to_admit(seq)
            if needed > self.cache.num_pages:
                self.waiting.popleft()
                self._fail(seq, f"kv pool has {self.cache.num_pages} blocks of {self.cache.page_size}; "
                                f"this sequence needs {needed}")
                continue
            if self.cache.free_slot_count() == 0:
                break
            self.cache.add_request(seq.id)
            shared = self.cache.attach_shared_prefix(seq.id, seq.tokens)
            if not self.cache.reserve(seq.id, needed * self.cache.page_size):
                self.cache.release(seq.id)      # gives back the shared pages and the slot
                break
            self.waiting.popleft()
            seq.computed = shared
            self.running.append(seq)
        self.stats.max_running = max(self.stats.max_running, len(self.running))

    # ------------------------------------------------------------------- planning
    def _preempt(self, seq: Sequence, preempted: list[Sequence]) -> None:
        self.running.remove(seq)
        self.cache.release(seq.id)
        seq.computed = 0
        self.stats.preemptions += 1
        self.stats.last_preempted_id = seq.id
        preempted.append(seq)

    def _fail(self, seq: Sequence, message: str) -> None:
        if seq in self.running:
            self.running.remove(seq)
            self.cache.release(seq.id)
        seq.result = Failure(message)
        self.finished[seq.id] = seq.result
        self.stats.requests_failed += 1

    def _plan(self, preempted: list[Sequence]) -> list[tuple[Sequence, int]]:
        """(sequence, tokens to run) for this iteration, pages reserved.  Oldest first; decoding
        sequences before prompt portions."""
        budget = self.config.max_num_batched_tokens
        chunk = self.config.prefill_chunk or budget
        order = sorted(self.running, key=lambda s: (not s.decoding, s.id))
        planned: list[tuple[Sequence, int]] = []
        for seq in order:
            if seq not in self.running or budget <= 0:
                continue
            count = 1 if seq.decoding else min(seq.remaining, budget, chunk)
            new_len = seq.computed + count
            while not self.cache.reserve(seq.id, new_len):
                needed = pages_for_len(new_len, self.cache.page_size)
                if needed > self.cache.num_pages:
                    self._fail(seq, f"kv pool has {self.cache.num_pages} blocks of {self.cache.page_size}; "
                                    f"this sequence needs {needed}")
                    break
                victim = max(self.running, key=lambda s: s.id)       # the newest (engine.rs:632-639)
                planned = [(s, n) for s, n in planned if s is not victim]
                self._preempt(victim, preempted)
                if victim is seq:
                    break
            if seq in self.running:
                planned.append((seq, count))
                budget -= count
        return planned

    # ----------------------------------------------------------------------- step
    def step(self) -> bool:
        """One iteration.  Returns False when there was nothing to run."""
        self._admit()
        if not self.running:
            return False
        preempted: list[Sequence] = []
        planned = self._plan(preempted)
        if planned:
            self._run(planned)
        self._note_peaks()
        # Oldest preempted sequence first, ahead of requests that never ran (engine.rs:369-376).
        for seq in sorted(preempted, key=lambda s: s.id, reverse=True):
            self.waiting.appendleft(seq)
        return bool(planned) or bool(preempted)

    def _run(self, planned: list[tuple[Sequence, int]]) -> None:
        entries, wanting = [], []
        for seq, count in planned:
            tokens = seq.tokens[seq.computed:seq.computed + count]
            completes = seq.computed + count == len(seq.tokens)
            wants = completes and seq.params.max_tokens > 0
            entries.append(StepEntry(seq.id, tokens, [count - 1] if wants else []))
            if wants:
                wanting.append(seq)
        started = time.perf_counter()
        logits = self.engine.step(entries)
        greedy_rows = [row for row, seq in enumerate(wanting) if seq.cursor.is_greedy]
        warm_rows = [row for row, seq in enumerate(wanting) if not seq.cursor.is_greedy]
        picked: dict[int, int] = {}
        if greedy_rows:
            for row, token in zip(greedy_rows, self.engine.argmax(logits, greedy_rows)):
                picked[row] = int(token)
        warm_logits = None
        if warm_rows and hasattr(self.engine, "sample"):
            # Drawn on the device: each request brings its own uniform number, so a draw does not depend on
            # who else is in the batch.
            cursors = [wanting[row].cursor for row in warm_rows]
            tokens = self.engine.sample(logits, warm_rows, [c.params.temperature for c in cursors],
                                        [c.params.top_p for c in cursors], [c.next_uniform() for c in cursors])
            for row, token in zip(warm_rows, tokens):
                picked[row] = int(token)
        elif warm_rows:
            warm_logits = self.engine.rows_to_host(logits, warm_rows)
        elapsed = time.perf_counter() - started
        self.stats.steps += 1
        self.stats.tokens_forwarded += sum(count for _, count in planned)
        n_decoding = sum(1 for seq, _ in planned if seq.decoding) or 1
        for seq, count in planned:
            if seq.decoding:
                seq.decode += elapsed / n_decoding     # shares add up to the step (engine.rs:909-916)
            else:
                seq.prefill += elapsed
            seq.computed += count
            if seq.computed - count < len(seq.prompt):      # the portion held prompt tokens
                self.cache.publish(seq.id, seq.prompt)
        for row, seq in enumerate(wanting):
            if row in picked:
                outcome = seq.cursor.push_token(picked[row], seq.token_bytes, seq.on_chunk)
            else:
                outcome = seq.cursor.push_logits(warm_logits[warm_rows.index(row)], seq.token_bytes, seq.on_chunk)
            self._after_sample(seq, outcome)
        for seq, _ in planned:
            if seq.result is None and seq.computed == len(seq.tokens) and seq.params.max_tokens == 0:
                self._finish(seq, seq.cursor.finish_without_sample(seq.on_chunk))

    def _after_sample(self, seq: Sequence, outcome) -> None:
        if isinstance(outcome, Sampled):
            self._finish(seq, outcome)
        else:
            seq.tokens.append(int(outcome))

    def _finish(self, seq: Sequence, done: Sampled) -> None:
        seq.result = Generated(done.tokens, done.text, done.chunks, done.reason, done.completion_tokens,
                               seq.prefill, seq.decode)
        self.finished[seq.id] = seq.result
        self.running.remove(seq)
        self.cache.release(seq.id)
        self.stats.requests_finished += 1

    def cancel(self, seq_id: int) -> None:
        """Stop a request before its next forward; what it sampled so far is its result."""
        for seq in list(self.running) + list(self.waiting):
            if seq.id == seq_id:
                if seq in self.running:
                    self._finish(seq, seq.cursor.snapshot(StopReason.Cancelled))
                else:
                    self.waiting.remove(seq)
                    done = seq.cursor.snapshot(StopReason.Cancelled)
                    self.finished[seq.id] = Generated(done.tokens, done.text, done.chunks, done.reason,
                                                      done.completion_tokens, seq.prefill, seq.decode)
                    self.stats.requests_finished += 1
                return

    def _note_peaks(self) -> None:
        for group in self.cache.groups:
            self.stats.peak_blocks = max(self.stats.peak_blocks, group.allocator.peak_live)
            self.stats.peak_occupied = max(self.stats.peak_occupied, group.allocator.peak_occupied)

    # ------------------------------------------------------------------------ run
    def run(self, max_steps: int | None = None) -> dict[int, Generated | Failure]:
        """Iterate until every request has finished; returns the results by request id."""
        steps = 0
        while self.has_work():
            progressed = self.step()
            steps += 1
            if not progressed and not self.running and self.waiting:
                # The front of the queue cannot be admitted into an empty batch: it never will be.
                seq = self.waiting.popleft()
                self._fail(seq, f"kv pool has {self.cache.num_pages} blocks of {self.cache.page_size}; "
                                f"this sequence needs {self._pages_to_admit(seq)}")
            if max_steps is not None and steps >= max_steps:
                break
        return self.finished

    def assert_idle(self) -> None:
        """With nothing live every count is zero and, cached pages reclaimed, every page is free
        (engine.rs:385-400)."""
        assert not self.running and not self.waiting
        assert not self.cache.requests
        for group in self.cache.groups:
            assert group.allocator.all_refcounts_zero(), "kv refcounts still held"
            group.allocator.reclaim_cached()
            assert group.allocator.free_count() == group.allocator.capacity(), "kv blocks still assigned"
        self.cache.check_invariants()
