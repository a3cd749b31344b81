"""Continuous-batching scheduler above the step function.

Policy follows qwen-server/src/engine.rs: a FIFO of waiting requests and a running batch;
admission looks at the front of the queue only and reserves pages for the whole prompt
(458-517); each iteration grows the running sequences oldest first and, when pages run out,
preempts the newest sequence, which gives back everything and is recomputed later (561-668);
preempted sequences return to the front of the queue, oldest first (369-376); a sequence that
cannot fit in the whole pool fails with a message (473-487, 670-685).

Beyond the reference, one iteration is a single mixed batch under a token budget: one token
for every decoding sequence first, then portions of prompts in order of arrival
(`SchedulerConfig.prompts_first` turns that round, as the reference orders an iteration, new
sequences prefilled before the batched decode, 788-805; under a budget the decoding sequences
then wait while prompts fill it, which the reference, having no budget, does not make them do).  A preempted
sequence is recomputed from its prompt and the tokens it sampled so far, and nothing is
sampled again for positions that already have a token.

The decisions (queue, admission, plan, preemption, every exchange with the cache manager) are
made by the C++ scheduler core (`csrc/host/scheduler_core.cpp`), which also owns the token lists;
this class runs the plan through the engine, samples, keeps stop conditions, texts and results.
"""
from __future__ import annotations

import ctypes
import dataclasses
import time
from typing import Callable

import numpy as np

from .. import host as _host
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
    decode_burst: int = 16       # greedy decode steps that may run back to back without the host in between
    # Who takes the token budget first.  False: decoding sequences, one token each, then portions of prompts: a
    # running request gets a token in every step whatever arrives.  True: portions of prompts, then decoding
    # sequences with what is left: they wait while prompts stand in line and then decode together in full
    # batches, fewer and cheaper steps for the same tokens when many requests arrive at once.
    prompts_first: bool = False


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
    prefix_hits: int = 0             # admissions that took over pages another request had computed
    prefix_tokens_reused: int = 0    # tokens those pages held (never forwarded again)
    steps: int = 0
    tokens_forwarded: int = 0


class QueueFull(RuntimeError):
    pass


@dataclasses.dataclass
class Failure:
    message: str


class Sequence:
    """What the host keeps of a sequence: its sampler, callbacks and timings.  Its tokens live in the core."""

    def __init__(self, seq_id: int, prompt_len: int, params: GenerateParams, token_bytes, on_chunk):
        self.id = seq_id
        self.prompt_len = prompt_len
        self.params = params
        self.cursor = SampleCursor(params)
        self.token_bytes = token_bytes
        self.on_chunk = on_chunk
        self.prefill = 0.0
        self.decode = 0.0
        self.result: Generated | Failure | None = None


_RUNNING, _WAITING, _MAX_RUNNING, _PREEMPTIONS, _LAST_PREEMPTED, _FRONT, _PAGES_TO_ADMIT, _COMPUTED, _N_TOKENS, \
    _IS_RUNNING, _PREFIX_HITS, _PREFIX_TOKENS = range(12)


class Scheduler:
    """Admits requests, cuts prompts into portions, decodes, finishes and frees.

    `engine` needs: `.cache` (a CacheManager), `.step(entries, reserve=False) -> logits`, `.argmax(logits, rows) ->
    list[int]`, `.max_positions`, and for warm requests `.sample(logits, rows, temperature, top_p, uniform)
    -> list[int]` or, without it, `.rows_to_host(logits, rows) -> float32 array` (drawn on the host then).
    """

    def __init__(self, engine, config: SchedulerConfig | None = None):
        self.engine = engine
        self.cache = engine.cache
        self.config = config or SchedulerConfig()
        self._lib = _host.lib()
        self._core = self._lib.ta_sched_new(self.cache._core, self.cache.num_pages, self.config.max_batch_size,
                                            self.config.max_num_batched_tokens, self.config.prefill_chunk or 0,
                                            1 if self.config.prompts_first else 0)
        if not self._core:
            raise ValueError("max_batch_size and max_num_batched_tokens must be positive")
        self._cache_core_owner = self.cache._core_owner      # the cache core outlives this scheduler's core
        self.sequences: dict[int, Sequence] = {}          # every sequence the core knows: waiting or running
        self.finished: dict[int, Generated | Failure] = {}
        self.stats = EngineStats()
        self._next_id = 1

    def __del__(self):
        if getattr(self, "_core", None):
            self._lib.ta_sched_delete(self._core)
            self._core = None

    def _get(self, what: int, seq_id: int = 0) -> int:
        return int(self._lib.ta_sched_get(self._core, what, seq_id))

    def _listed(self, which: int) -> list[Sequence]:
        out = (ctypes.c_int64 * max(1, len(self.sequences)))()
        count = self._lib.ta_sched_list(self._core, which, out)
        return [self.sequences[i] for i in out[:count]]

    @property
    def running(self) -> list[Sequence]:
        """The running sequences in order of admission."""
        return self._listed(0)

    @property
    def waiting(self) -> list[Sequence]:
        """The queue, its front first."""
        return self._listed(1)

    # ------------------------------------------------------------------- requests
    def add_request(self, prompt: list[int], params: GenerateParams | None = None,
                    token_bytes: Callable[[int], bytes] = _no_bytes,
                    on_chunk: Callable[[str], Control] = _go_on) -> int:
        """Queue a request; returns its id.  Problems with the request itself are recorded as a failed
        result under that id (as the reference answers them on the request's own channel)."""
        params = params or GenerateParams()
        if self._get(_WAITING) >= self.config.max_waiting:
            raise QueueFull(f"{self._get(_WAITING)} requests are already waiting")
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
            seq = Sequence(seq_id, len(prompt), params, token_bytes, on_chunk)
        except ValueError as err:
            self._fail_new(seq_id, str(err))
            return seq_id
        keep, pointer = _host.int_array(list(prompt))
        self._lib.ta_sched_enqueue(self._core, seq_id, pointer, len(keep))
        self.sequences[seq_id] = seq
        return seq_id

    def _fail_new(self, seq_id: int, message: str) -> None:
        self.finished[seq_id] = Failure(message)
        self.stats.requests_failed += 1

    def has_work(self) -> bool:
        return bool(self.sequences)

    def _pool_message(self, pages_needed: int) -> str:
        return (f"kv pool has {self.cache.num_pages} blocks of {self.cache.page_size}; "
                f"this sequence needs {pages_needed}")

    def _record_failure(self, seq_id: int, message: str) -> None:
        """The core has already dropped the sequence and given back what it held."""
        seq = self.sequences.pop(seq_id)
        seq.result = Failure(message)
        self.finished[seq_id] = seq.result
        self.stats.requests_failed += 1

    # ----------------------------------------------------------------------- step
    def step(self) -> bool:
        """One iteration: the core admits, plans (pages reserved, the newest sequence preempted when they run
        out) and requeues; the plan is then run as one batch.  Returns False when nothing changed: nothing ran,
        nothing was preempted and nothing failed (a sequence that fails gives back its pages, so the queue's
        front may well be admitted in the next iteration)."""
        room = max(1, len(self.sequences))
        planned = (ctypes.c_int64 * (4 * room))()
        preempted = (ctypes.c_int64 * room)()
        failed = (ctypes.c_int64 * (2 * room))()
        counts = [ctypes.c_int32(0) for _ in range(3)]
        status = self._lib.ta_sched_plan_step(self._core, room, planned, ctypes.byref(counts[0]), preempted,
                                              ctypes.byref(counts[1]), failed, ctypes.byref(counts[2]))
        if status != 0:
            raise RuntimeError("the scheduler core's plan did not fit its buffers")
        n_planned, n_preempted, n_failed = (c.value for c in counts)
        for i in range(n_failed):
            self._record_failure(int(failed[2 * i]), self._pool_message(int(failed[2 * i + 1])))
        plan = [(self.sequences[int(planned[4 * i])], int(planned[4 * i + 1]), int(planned[4 * i + 2]),
                 bool(planned[4 * i + 3])) for i in range(n_planned)]
        if plan:
            burst = self._burst_length(plan)
            if burst > 1:
                self._run_burst(plan, burst)
            else:
                self._run(plan)
        self._note_peaks()
        return bool(plan) or n_preempted > 0 or n_failed > 0

    def _tokens(self, seq_id: int, first: int, count: int):
        """The sequence's tokens first .. first + count - 1: a list, or (long portions) an array, which the engine
        takes as it is."""
        out = (ctypes.c_int32 * max(1, count))()
        self._lib.ta_sched_tokens(self._core, seq_id, first, count, out)
        if count > 64:
            return np.ctypeslib.as_array(out)[:count].astype(np.int64)
        return list(out[:count])

    def _run(self, plan: list[tuple[Sequence, int, int, bool]]) -> None:
        entries, wanting = [], []
        for seq, first, count, completes in plan:
            wants = completes and seq.params.max_tokens > 0
            entries.append(StepEntry(seq.id, self._tokens(seq.id, first, count), [count - 1] if wants else []))
            if wants:
                wanting.append(seq)
        started = time.perf_counter()
        logits = self.engine.step(entries, reserve=False)       # the plan reserved every page
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
        self.stats.tokens_forwarded += sum(count for _, _, count, _ in plan)
        decoding = [first >= seq.prompt_len and count == 1 for seq, first, count, _ in plan]
        n_decoding = sum(decoding) or 1
        for (seq, _, count, _), is_decoding in zip(plan, decoding):
            if is_decoding:
                seq.decode += elapsed / n_decoding     # shares add up to the step (engine.rs:909-916)
            else:
                seq.prefill += elapsed
            self._lib.ta_sched_commit(self._core, seq.id, count)     # full prompt pages become shareable
        for row, seq in enumerate(wanting):
            if row in picked:
                outcome = seq.cursor.push_token(picked[row], seq.token_bytes, seq.on_chunk)
            else:
                outcome = seq.cursor.push_logits(warm_logits[warm_rows.index(row)], seq.token_bytes, seq.on_chunk)
            if isinstance(outcome, Sampled):
                self._finish(seq, outcome)
            else:
                self._lib.ta_sched_append_token(self._core, seq.id, int(outcome))
        for seq, _, _, completes in plan:
            if seq.result is None and completes and seq.params.max_tokens == 0:
                self._finish(seq, seq.cursor.finish_without_sample(seq.on_chunk))

    # ---------------------------------------------------------------------- bursts
    def _burst_length(self, plan: list[tuple[Sequence, int, int, bool]]) -> int:
        """How many decode steps may follow each other on the device without a decision of the host between them:
        more than one only when the step is nothing but decoding, greedy or drawn on the device (the ids a step
        picks feed the next one there, `Engine.decode_greedy` and `Engine.decode_sampled`), nothing waits that could join, no sequence reaches its last token before the
        burst's last step, and the pages for all those tokens of all sequences are there now (a burst the pool
        cannot hold whole is halved until it can)."""
        burst = min(self.config.decode_burst, 64)
        if burst < 2 or not getattr(self.engine, "use_graphs", False) or not hasattr(self.engine, "decode_greedy"):
            return 1
        if (not all(seq.cursor.is_greedy for seq, _, _, _ in plan)
                and not (hasattr(self.engine, "decode_sampled") and hasattr(self.engine, "sample"))):
            return 1                     # draws that only the host can make: one step at a time
        if self._get(_WAITING) and len(plan) < self.config.max_batch_size:
            return 1                     # the queue's front waits for pages: a finished sequence should let it in at once
        if len(plan) != self._get(_RUNNING):
            return 1                     # the token budget left a running sequence out of this step: it is next
        for seq, first, count, completes in plan:
            if count != 1 or first < seq.prompt_len or not completes:
                return 1
            burst = min(burst, seq.params.max_tokens - seq.cursor.produced)
        # The pages for all those tokens of all the sequences are taken together or not at all: a burst that only
        # some sequences got their pages for would leave those holding pages they do not need yet, and the next
        # plan might then find none for another sequence's single token and preempt, where single steps would
        # still have fitted.  A burst the pool cannot hold is halved until it can.
        while burst >= 2:
            missing = [0] * len(self.cache.groups)
            for seq, first, _, _ in plan:
                for group, pages in enumerate(self.cache.pages_missing(seq.id, first + burst)):
                    missing[group] += pages
            if all(pages <= group.allocator.available() for pages, group in zip(missing, self.cache.groups)):
                break
            burst //= 2
        if burst < 2:
            return 1
        for seq, first, _, _ in plan:
            if not self.cache.reserve(seq.id, first + burst):       # tokens first .. first + burst - 1 get their pages
                return 1                  # (cannot happen after the count above; pages taken so far are theirs early, no more)
        return burst

    def _run_burst(self, plan: list[tuple[Sequence, int, int, bool]], burst: int) -> None:
        """`burst` decode steps of the planned sequences back to back, greedy or drawn on the device (the generator
        of a sequence that draws gives one uniform number for every step that is launched).  Ids reach the host one
        step late; when one of them ends a sequence (end-of-sequence id, stop string, the caller's callback), the
        step after it is already on its way: the others keep its tokens, the finished sequence's one is dropped."""
        seqs = [seq for seq, _, _, _ in plan]
        tokens = [self._tokens(seq.id, first, 1)[0] for seq, first, _, _ in plan]
        handled = 0
        started = time.perf_counter()

        def take(ids) -> bool:
            nonlocal handled, started
            now = time.perf_counter()
            elapsed, started = now - started, now
            handled += 1
            live = [seq for seq in seqs if seq.result is None]
            go_on = True
            self.stats.steps += 1
            self.stats.tokens_forwarded += len(live)
            for seq, token in zip(seqs, ids):
                if seq.result is not None:
                    continue              # ended earlier in this burst: what the step already under way picked for it is dropped
                seq.decode += elapsed / len(live)
                self._lib.ta_sched_commit(self._core, seq.id, 1)
                outcome = seq.cursor.push_token(int(token), seq.token_bytes, seq.on_chunk)
                if isinstance(outcome, Sampled):
                    self._finish(seq, outcome)
                    go_on = False
                else:
                    self._lib.ta_sched_append_token(self._core, seq.id, int(outcome))
            return go_on

        rids = [seq.id for seq in seqs]
        cursors = [seq.cursor for seq in seqs]
        if all(c.is_greedy for c in cursors):
            picked = self.engine.decode_greedy(rids, tokens, burst, on_step=lambda k, ids: take(ids))
        else:
            # (A greedy sequence among them has temperature 0, keeps the greedy pick and has no number to give.)
            draw = lambda k: ([c.params.temperature for c in cursors], [c.params.top_p for c in cursors],
                              [0.5 if c.is_greedy else c.next_uniform() for c in cursors])
            picked = self.engine.decode_sampled(rids, tokens, burst, draw, on_step=lambda k, ids: take(ids))
        for ids in picked[handled:]:      # the step that was under way when a sequence ended
            take(ids)

    def _finish(self, seq: Sequence, done: Sampled) -> None:
        seq.result = Generated(done.tokens, done.text, done.chunks, done.reason, done.completion_tokens,
                               seq.prefill, seq.decode)
        self.finished[seq.id] = seq.result
        self._lib.ta_sched_finish(self._core, seq.id)       # pages and the slot go back
        del self.sequences[seq.id]
        self.stats.requests_finished += 1

    def cancel(self, seq_id: int) -> None:
        """Stop a request before its next forward; what it sampled so far is its result."""
        seq = self.sequences.get(seq_id)
        if seq is not None:
            self._finish(seq, seq.cursor.snapshot(StopReason.Cancelled))

    def _note_peaks(self) -> None:
        self.stats.max_running = self._get(_MAX_RUNNING)
        self.stats.preemptions = self._get(_PREEMPTIONS)
        self.stats.last_preempted_id = self._get(_LAST_PREEMPTED)
        self.stats.prefix_hits = self._get(_PREFIX_HITS)
        self.stats.prefix_tokens_reused = self._get(_PREFIX_TOKENS)
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
            if not progressed and self._get(_RUNNING) == 0 and self._get(_WAITING) > 0:
                # The front of the queue cannot be admitted into an empty batch: it never will be.
                front = self._get(_FRONT)
                needed = self._get(_PAGES_TO_ADMIT, front)
                self._lib.ta_sched_finish(self._core, front)
                self._record_failure(front, self._pool_message(needed))
            if max_steps is not None and steps >= max_steps:
                break
        return self.finished

    def assert_idle(self) -> None:
        """With nothing live every count is zero and, cached pages reclaimed, every page is free
        (engine.rs:385-400)."""
        assert self._get(_RUNNING) == 0 and self._get(_WAITING) == 0 and not self.sequences
        assert not self.cache.requests
        for group in self.cache.groups:
            assert group.allocator.all_refcounts_zero(), "kv refcounts still held"
            group.allocator.reclaim_cached()
            assert group.allocator.free_count() == group.allocator.capacity(), "kv blocks still assigned"
        self.cache.check_invariants()
