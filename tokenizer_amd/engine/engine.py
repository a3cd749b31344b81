"""The engine: a model, its cache and the one step function everything else is built on."""
from __future__ import annotations

import numpy as np
import torch

from ..cache import CacheManager, CachePools, OutOfPages
from ..config import load_config
from ..config.base import ModelConfig
from ..config.registry import get_architecture
from ..parts import LayerCache, Runtime, build_model, cache_needs, expected_tensors
from ..weights import load_weights, random_tensors, stored_form
from .batch import StepEntry, build_context, filled_counts

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def resolve_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype must be bfloat16 or float32, not {dtype!r}") from None


class Model:
    """A configuration, its `ModelSpec` and the built parts with their weights on the device."""

    def __init__(self, config: ModelConfig, tensors: dict[str, torch.Tensor], dtype, device="cuda:0", ops=None):
        from ..kernels import get_ops
        self.config = config
        self.dtype = resolve_dtype(dtype)
        self.device = torch.device(device)
        self.spec = get_architecture(config.architecture).build_spec(config)
        self.runtime = Runtime(self.dtype, self.device, ops if ops is not None else get_ops())
        self.decoder = build_model(self.spec, tensors, self.runtime)     # in the frame the spec names
        self.cache_needs = cache_needs(self.spec)

    @property
    def vocab_size(self) -> int:
        return self.spec.vocab_size

    @property
    def max_positions(self) -> int:
        return self.spec.max_positions


def load_model(folder: str, dtype="bfloat16", device="cuda:0", ops=None) -> Model:
    """Build the model that `folder/config.json` names, with the weights of `folder/model.safetensors`."""
    config = load_config(folder)
    spec = get_architecture(config.architecture).build_spec(config)
    tensors = load_weights(folder, expected_tensors(spec), resolve_dtype(dtype), device)
    return Model(config, tensors, dtype, device, ops)


def random_model(config: ModelConfig, seed: int, dtype="bfloat16", device="cuda:0", ops=None) -> Model:
    """The model of `config` with the weights the random-weights mode would write for `seed`."""
    spec = get_architecture(config.architecture).build_spec(config)
    expected = expected_tensors(spec)
    compute = resolve_dtype(dtype)
    tensors = {}
    for name, tensor in random_tensors(expected, seed).items():
        tensors[name] = stored_form(tensor, expected[name], compute).to(device).contiguous()
    return Model(config, tensors, dtype, device, ops)


class StepGraph:
    """One captured HIP graph of a step of one shape (a decode step: so many requests with one token each; any
    other step: the counts of tokens, entries, wanted places, prompt tiles and single rows its description is
    filled up to), contexts of up to `bucket` tokens.  The batch's tables live in fixed buffers that are refilled
    before every replay; the graph ends with the greedy pick, so ids are ready without a further launch."""

    def __init__(self, engine: "Engine", entries: list[StepEntry], bucket: int):
        self.bucket = bucket
        self.width = -(-bucket // engine.cache.page_size)
        device = engine.model.device
        probe = build_context(entries, engine.cache, device, table_width=self.width, fill=True)
        size = sum(t.numel() for t in (probe.token_ids, probe.positions, probe.entry_of_token, probe.cu_q,
                                       probe.first_position, probe.state_slots, probe.want_rows, probe.q_tiles,
                                       probe.decode_rows))
        size += sum(t.numel() for t in probe.slots) + sum(t.numel() for t in probe.block_tables)
        self.host = torch.empty(size, dtype=torch.int32).pin_memory()
        self.dev = torch.empty(size, dtype=torch.int32, device=device)
        self.ctx = build_context(entries, engine.cache, device, table_width=self.width, into=(self.host, self.dev), fill=True)
        self.ctx.max_position = bucket - 1          # what the kernels' launch sizes are planned for
        ops = engine.model.runtime.ops
        before = getattr(ops, "capturing", False)
        ops.capturing = True                        # kernels are chosen by their time on the device alone
        try:
            side = torch.cuda.Stream(device=device)
            side.wait_stream(torch.cuda.current_stream(device))
            with torch.cuda.stream(side):           # one eager run first, so that nothing is set up under capture
                engine.model.decoder.forward(self.ctx, engine.layer_caches)
            torch.cuda.current_stream(device).wait_stream(side)
            torch.cuda.synchronize(device)
            # A plain decode step (one token per request, its logits wanted) may end by turning its own description
            # into the next step's on the device (`Ops.argmax_next_step`): in a run of such steps the host then
            # has nothing to upload between them, as long as what it would upload is what the device holds already.
            ctx = self.ctx
            self.advances = (engine.NEXT_STEP_ON_DEVICE
                             and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries)
                             and len(ctx.slots) <= getattr(ops, "NEXT_STEP_GROUPS", -1))
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, pool=engine.graph_pool):
                self.logits = engine.model.decoder.forward(self.ctx, engine.layer_caches)
                if self.advances:
                    self.ids = ops.argmax_next_step(self.logits, ctx.token_ids, ctx.positions, ctx.first_position,
                                                    ctx.slots, ctx.block_tables, ctx.page_size)
                else:
                    self.ids = ops.argmax(self.logits) if self.logits.shape[0] else None
        finally:
            ops.capturing = before
        self.uploaded = None
        self.uploads = 0                            # times the description went to the device
        self.on_device = None                       # what the device's copy of the description holds, where that is known
        self.last_used = 0
        self.draws = None                           # captured graphs of the sampler over these logits, made on demand

    def draw_on_device(self, engine: "Engine", temperature: list[float], top_p: list[float], uniform: list[float],
                       any_cut: bool) -> torch.Tensor:
        """Temperature / nucleus draws for every row of this graph's logits, left on the device (int32, one per
        row; the rows past the given ones only fill the step up): the sampler's twenty small launches are captured
        once (per kind: with or without the rounds of the nucleus cut) and replayed.  Nothing waits for the result
        here."""
        rows = self.logits.shape[0]
        given = len(temperature)
        fill = [1.0] * (rows - given)
        temperature, top_p, uniform = list(temperature) + fill, list(top_p) + fill, list(uniform) + [0.5] * (rows - given)
        if self.draws is None:
            self.draws = {}
            self.draw_host = torch.empty((3, rows), dtype=torch.float32).pin_memory()
            self.draw_params = torch.empty((3, rows), dtype=torch.float32, device=self.logits.device)
            self.draw_ids = torch.zeros(rows, dtype=torch.int32, device=self.logits.device)
            self.draw_uploaded = torch.cuda.Event()
        self.draw_uploaded.synchronize()              # the last draw's numbers have left the pinned buffer
        self.draw_host.copy_(torch.tensor([temperature, top_p, uniform], dtype=torch.float32))
        self.draw_params.copy_(self.draw_host, non_blocking=True)
        self.draw_uploaded.record()
        ops = engine.model.runtime.ops
        launch = lambda: ops.sample(self.logits, self.draw_params[0], self.draw_params[1], self.draw_params[2],
                                    out=self.draw_ids, any_cut=any_cut)
        captured = self.draws.get(any_cut)
        if captured is None:
            launch()                                      # once eagerly: the draw of this call, and a warm-up
            torch.cuda.synchronize(self.logits.device)
            captured = torch.cuda.CUDAGraph()
            with torch.cuda.graph(captured, pool=engine.graph_pool):
                launch()
            self.draws[any_cut] = captured
        else:
            captured.replay()
        return self.draw_ids

    def draw(self, engine: "Engine", temperature: list[float], top_p: list[float], uniform: list[float],
             any_cut: bool) -> list[int]:
        """The same draws, brought to the host: one id for each of the given rows."""
        ids = self.draw_on_device(engine, temperature, top_p, uniform, any_cut)
        return [int(v) for v in ids.cpu().tolist()][:len(temperature)]

    def run(self, engine: "Engine", entries: list[StepEntry], tokens_on_device: torch.Tensor | None = None) -> torch.Tensor:
        """Pack the batch's description into the fixed buffers again and replay.  `tokens_on_device`: the token
        ids come from this int32 tensor on the device (the ids an earlier replay picked), not from the entries."""
        if self.uploaded is not None:
            self.uploaded.synchronize()                 # the last upload has left the pinned buffer
        else:
            self.uploaded = torch.cuda.Event()
        manager = engine.cache
        total, _, _, _ = manager.pack_batch([e.rid for e in entries], [e.packed_tokens() for e in entries],
                                            [e.want for e in entries], self.host.numpy(), self.width,
                                            filled_counts([len(e.tokens) for e in entries], [len(e.want) for e in entries]))
        if total != self.host.numel():
            raise ValueError("the packed batch does not fit the graph's buffers")
        count = len(entries)
        packed = self.host.numpy()
        # (The token ids lead the buffer.  A step that takes them from this graph's last pick finds them in place.)
        in_place = (self.advances and tokens_on_device is self.ids and self.on_device is not None
                    and np.array_equal(packed[count:], self.on_device[count:]))
        if not in_place:
            self.dev.copy_(self.host, non_blocking=True)
            self.uploaded.record()
            self.uploads += 1
            if tokens_on_device is not None:
                self.dev[:count].copy_(tokens_on_device[:count], non_blocking=True)
        self.graph.replay()
        if self.advances:
            self.on_device = next_decode_description(packed, count, manager.page_size, self.width, len(self.ctx.slots))
        return self.logits


def next_decode_description(packed: np.ndarray, count: int, page_size: int, width: int, n_groups: int) -> np.ndarray:
    """What `Ops.argmax_next_step` makes of a plain decode step's description (all but the token ids, which only
    the device knows): the layout is `CacheCore::pack_batch`'s for `count` entries of one token each, with tables of
    `width` pages for each of the `n_groups` cache groups."""
    after = packed.copy()
    positions = after[count:2 * count]
    positions += 1
    at = 3 * count + count + 1                             # past token ids, positions, entries of tokens, first rows
    after[at:at + count] += 1                              # first positions
    at += 4 * count                                        # past state slots, wanted rows (no tiles), single rows
    rows = np.arange(count)
    for _ in range(n_groups):
        table = after[at + count:at + count + count * width].reshape(count, width)
        page = table[rows, np.minimum(positions // page_size, width - 1)]
        after[at:at + count] = np.where(page < 0, -1, page * page_size + positions % page_size)
        at += count + count * width
    if at != after.size:
        raise ValueError("not the description of a step of single tokens")
    return after


class Engine:
    """Owns the cache of one model and runs steps.

    `step(entries)` runs exactly the tokens it is given, as one batch, against what earlier steps
    left in the cache, and returns float32 logits at the wanted places, in the order of the
    entries and of each entry's `want`.
    """

    GRAPH_BUCKET = 512      # graphs are captured per shape of the step and per this many tokens of context
    STEP_GRAPHS = 64        # how many graphs of other steps than plain decode steps are kept
    GRAPH_IDLE_STEPS = 2000  # a kept graph makes room for another only after this many steps without a replay
    GRAPH_TOKENS = 2048     # steps with more tokens than this are not captured: the device is the slower side
    GRAPH_AFTER = 3         # a shape is captured when it comes up for this many times ...
    SHAPES_REMEMBERED = 64  # ... among this many shapes seen last
    # Whether the graphs of plain decode steps end with the kernel that writes the next step's description in place
    # (see `StepGraph`): a decode step then needs neither the upload of its description nor the copy of the picked ids,
    # two small copies of about 8 us together before a step of 0.8 to 1.5 ms at 0.5B sizes.  Off: such a graph must
    # never be replayed without the host's check in `StepGraph.run` before it (each replay moves every request one
    # position on, and positions that run past the pages a request holds make the attention read addresses that are
    # not there), which is so for every replay in this package; it has been run through the tests that name it
    # only, not through the whole suite and the serving workloads.
    NEXT_STEP_ON_DEVICE = False

    def __init__(self, model: Model, num_pages: int | None = None, page_size: int = 16, max_requests: int = 8,
                 max_tokens: int | None = None, prefix_cache: bool = False, use_graphs: bool | None = None,
                 num_blocks: int | None = None, max_batch_size: int | None = None,
                 max_num_batched_tokens: int = 2048):
        """`num_blocks` and `max_batch_size` are the reference's names (qwen-server/src/lib.rs:33-56) for
        `num_pages` and `max_requests`; `max_num_batched_tokens` is the token budget of `run()`.  Without
        `num_pages` the pool is made for `max_tokens`: the most tokens that live requests hold at any time, each
        request's count rounded up to a multiple of 64."""
        num_pages = num_blocks if num_pages is None else num_pages
        max_requests = max_batch_size if max_batch_size is not None else max_requests
        self.max_num_batched_tokens = max_num_batched_tokens
        self._scheduler = None
        if num_pages is None:
            if max_tokens is None:
                raise ValueError("give num_pages or max_tokens")
            # `max_tokens` counts every live request's tokens rounded up to a multiple of 64.  Pages whose size
            # does not divide 64 round each request up on their own: at worst one page more per further request.
            num_pages = -(-max_tokens // page_size) + (max_requests - 1 if 64 % page_size else 0)
        self.model = model
        self.cache = CacheManager(model.cache_needs, num_pages, page_size, max_requests, prefix_cache)
        self.pools = CachePools(self.cache, model.cache_needs, model.dtype, model.device)
        self.layer_caches = []
        for entry in model.spec.schedule:
            source = entry.layer if entry.cache_of is None else entry.cache_of
            k_pages, v_pages = self.pools.layer_pages(source)
            self.layer_caches.append(LayerCache(group=self.cache.group_of_layer[source], k_pages=k_pages,
                                                v_pages=v_pages, state=self.pools.states.get(source),
                                                writes=entry.cache_of is None))
        self.steps = 0
        self._landing: dict[int, tuple] = {}     # pinned rows and events of `decode_greedy` / `decode_sampled`, by batch size
        self.steps_replayed = 0      # steps (decode steps and others) that replayed a captured graph
        self.graphs_captured = 0
        # Decode steps (one token per request, its logits wanted) and other steps whose shape recurs replay a
        # captured graph; the logits of a step stay valid until the next step.
        self.use_graphs = (model.device.type == "cuda") if use_graphs is None else use_graphs
        self.use_graphs = self.use_graphs and model.decoder.graph_safe
        self.graphs: dict[tuple, StepGraph] = {}
        self._shapes_seen: dict[tuple, int] = {}
        self.graph_pool = torch.cuda.graph_pool_handle() if self.use_graphs else None
        self._graph_result: StepGraph | None = None

    @property
    def max_positions(self) -> int:
        return self.model.max_positions

    # ------------------------------------------------------------------- sampling
    def argmax(self, logits: torch.Tensor, rows: list[int] | None = None) -> list[int]:
        """Greedy ids of the given rows of a step's logits, picked on the device."""
        graph = self._graph_result
        if graph is not None and self._is_result_of(logits, graph) and graph.ids is not None:
            picked = graph.ids.cpu().tolist()[:logits.shape[0]]    # the graph already picked them (and for the rows it was filled up with)
        else:
            picked = self.model.runtime.ops.argmax(logits).cpu().tolist()
        return picked if rows is None else [picked[row] for row in rows]

    def sample(self, logits: torch.Tensor, rows: list[int], temperature: list[float], top_p: list[float],
               uniform: list[float]) -> list[int]:
        """Temperature / nucleus draws for the given rows of a step's logits, on the device; one uniform
        number per row (from the request's own generator).  Draws for all rows of a replayed step's logits
        replay a captured graph of the sampler's launches as well."""
        device = logits.device
        any_cut = any(p < 1.0 for p in top_p)
        graph = self._graph_result
        if graph is not None and self._is_result_of(logits, graph) and rows == list(range(logits.shape[0])):
            return graph.draw(self, temperature, top_p, uniform, any_cut)
        picked = logits if rows == list(range(logits.shape[0])) else logits[torch.tensor(rows, device=device)]
        # One copy to the device for the three vectors.
        packed = torch.tensor([temperature, top_p, uniform], dtype=torch.float32).to(device, non_blocking=True)
        ids = self.model.runtime.ops.sample(picked.contiguous(), packed[0], packed[1], packed[2], any_cut=any_cut)
        return [int(v) for v in ids.cpu().tolist()]

    @staticmethod
    def _is_result_of(logits: torch.Tensor, graph: "StepGraph") -> bool:
        """Whether `logits` are the rows a replay of `graph` left (all of them, or the leading ones: those of the
        step's real entries)."""
        return logits is graph.logits or (logits.data_ptr() == graph.logits.data_ptr() and logits.shape[1:] == graph.logits.shape[1:]
                                          and logits.shape[0] <= graph.logits.shape[0])

    def rows_to_host(self, logits: torch.Tensor, rows: list[int]):
        return logits[rows].float().cpu().numpy()

    def decode_greedy(self, rids: list, tokens: list[int], n_steps: int, on_step=None) -> list[list[int]]:
        """`n_steps` greedy decode steps for the live requests `rids`, whose next tokens are `tokens`; returns the
        ids picked at every step, `n_steps` lists in the order of `rids`.

        The steps run back to back on the device: the ids a step picks feed the next step there, and the next
        step is launched before they have reached the host, which reads them one step late.  So the host's work
        on a step (tables, launch) hides behind the device's work on the step before.  `on_step(k, ids)` is
        called as each step's ids arrive; if it returns False the run ends after the step already launched (whose
        ids are still returned: the caller drops what it does not want; the cache holds those tokens too).
        Without captured graphs the steps run one by one through `step`."""
        return self._decode_run(rids, tokens, n_steps, on_step, None)

    def decode_sampled(self, rids: list, tokens: list[int], n_steps: int, draw, on_step=None) -> list[list[int]]:
        """The same run of decode steps with temperature / nucleus draws in place of the greedy pick.  `draw(k)`
        gives step k's (temperature, top_p, uniform) lists, one number of each per request; it is asked when step
        k is launched, once for every step that runs (so a request's generator hands out exactly one uniform
        number per token it is given, also when the run ends early).  A request whose temperature is 0 keeps the
        greedy pick (its other two numbers are not looked at)."""
        return self._decode_run(rids, tokens, n_steps, on_step, draw)

    @staticmethod
    def _warm_numbers(temperature, top_p, uniform):
        """The sampler's numbers for a step in which rows with temperature 0 take the greedy pick instead: those
        rows are drawn with harmless numbers and their draws thrown away.  Returns the lists and which rows are
        greedy."""
        greedy = [t == 0 for t in temperature]
        if not any(greedy):
            return list(temperature), list(top_p), list(uniform), greedy
        return ([1.0 if g else t for g, t in zip(greedy, temperature)], [1.0 if g else p for g, p in zip(greedy, top_p)],
                [0.5 if g else u for g, u in zip(greedy, uniform)], greedy)

    def _decode_run(self, rids: list, tokens: list[int], n_steps: int, on_step, draw) -> list[list[int]]:
        if n_steps <= 0:
            return []
        if len(rids) != len(tokens) or not rids:
            raise ValueError("one next token per request")
        count = len(rids)
        if not self.use_graphs:
            picked, current = [], list(tokens)
            for k in range(n_steps):
                logits = self.step([StepEntry(rid, [int(t)], [0]) for rid, t in zip(rids, current)])
                current = self.argmax(logits)
                if draw is not None:
                    temperature, top_p, uniform, greedy = self._warm_numbers(*draw(k))
                    drawn = self.sample(logits, list(range(count)), temperature, top_p, uniform)
                    current = [pick if g else token for g, pick, token in zip(greedy, current, drawn)]
                picked.append(list(current))
                if on_step is not None and on_step(k, picked[-1]) is False:
                    break
            return picked
        # (Two pinned rows for the ids on their way to the host and an event for each, kept from run to run: pinning
        # memory costs as much as several steps of a small model.)
        if count not in self._landing:
            self._landing[count] = ([torch.empty(count, dtype=torch.int32).pin_memory() for _ in range(2)],
                                    [torch.cuda.Event(), torch.cuda.Event()])
        landing, arrived = self._landing[count]
        picked: list[list[int]] = []
        previous: torch.Tensor | None = None           # where the step before left its ids, on the device
        greedy_rows, greedy_mask = None, None          # which requests keep the greedy pick in a run with draws
        go_on = True
        for k in range(n_steps):
            # Only the first step's token ids are known here; later steps take theirs from the step before.
            entries = [StepEntry(rid, [int(tokens[i]) if k == 0 else 0], [0]) for i, rid in enumerate(rids)]
            self.validate(entries)
            self.reserve(entries)
            graph = self._graph_for(entries)
            graph.run(self, entries, tokens_on_device=previous)
            for entry in entries:
                self.cache.advance(entry.rid, self.cache.seq_len(entry.rid) + 1)
            self.steps += 1
            if draw is None:
                previous = graph.ids
            else:
                temperature, top_p, uniform, greedy = self._warm_numbers(*draw(k))
                previous = graph.draw_on_device(self, temperature, top_p, uniform, any(p < 1.0 for p in top_p))
                if any(greedy):
                    if greedy != greedy_rows:
                        greedy_rows, greedy_mask = greedy, torch.tensor(greedy, device=previous.device)
                    previous = torch.where(greedy_mask, graph.ids[:count], previous[:count])
            landing[k % 2].copy_(previous[:count], non_blocking=True)   # queued before the next replay overwrites the ids
            arrived[k % 2].record()
            if k > 0:
                arrived[(k - 1) % 2].synchronize()
                picked.append(landing[(k - 1) % 2].tolist())
                if on_step is not None and on_step(k - 1, picked[-1]) is False:
                    go_on = False
            if not go_on:
                break
        last = len(picked)
        arrived[last % 2].synchronize()
        picked.append(landing[last % 2].tolist())
        if on_step is not None and go_on:
            on_step(last, picked[-1])
        self._graph_result = None
        return picked

    @staticmethod
    def _shape_of(entries: list[StepEntry]):
        """What fixes the layout of a step's tables and the sizes of its launches: the number of entries for a
        plain decode step; for a step of single tokens with other wishes, those; else the counts its description is
        filled up to (`filled_counts`), which steps that differ a little have in common."""
        if all(len(e.tokens) == 1 for e in entries):
            if all(list(e.want) == [0] for e in entries):
                return len(entries)
            return ("single",) + tuple(len(e.want) for e in entries)
        return ("filled",) + filled_counts([len(e.tokens) for e in entries], [len(e.want) for e in entries])

    def _graph_key(self, entries: list[StepEntry]) -> tuple:
        longest = max(self.cache.seq_len(e.rid) + len(e.tokens) for e in entries)
        # (The bucket is what the kernels' launch shapes are planned for, with any page size: an eager step plans
        # for its context rounded up in the same way, so both cut their sums alike.)
        bucket = -(-longest // self.GRAPH_BUCKET) * self.GRAPH_BUCKET
        return (self._shape_of(entries), bucket)

    def _graph_for(self, entries: list[StepEntry]) -> "StepGraph":
        key = self._graph_key(entries)
        graph = self.graphs.get(key)
        if graph is None:
            graph = StepGraph(self, entries, key[1])       # its first eager run and the capture write the same
            self.graphs[key] = graph                         # keys and values the replay writes again
            self.graphs_captured += 1
        self.steps_replayed += 1
        graph.last_used = self.steps
        return graph

    def _room_for_a_graph(self) -> bool:
        """Graphs of other steps than plain decode steps are kept up to `STEP_GRAPHS`; beyond that one makes room
        only if it has not been replayed for `GRAPH_IDLE_STEPS` steps (else a cycle of more shapes than graphs
        would capture every one of them again and again, which costs far more than running them eagerly)."""
        others = [key for key in self.graphs if not isinstance(key[0], int)]
        if len(others) < self.STEP_GRAPHS:
            return True
        oldest = min(others, key=lambda key: self.graphs[key].last_used)
        if self.steps - self.graphs[oldest].last_used < self.GRAPH_IDLE_STEPS:
            return False
        del self.graphs[oldest]
        return True

    def _replays(self, entries: list[StepEntry]) -> bool:
        """Whether this step replays a captured graph.  Plain decode steps always do.  Other steps (portions of
        prompts, mixed batches) do once their shape has come up `GRAPH_AFTER` times among the last
        `SHAPES_REMEMBERED` shapes: for short steps the host's launches, not the device, set the pace, and some
        shapes recur at once (a prompt cut into equal portions, a full token budget of equal prompts), while
        most mixes of a busy server never come again and are not worth a capture."""
        if not self.use_graphs:
            return False
        key = self._graph_key(entries)
        if isinstance(key[0], int) or key in self.graphs:
            return True
        if sum(len(e.tokens) for e in entries) > self.GRAPH_TOKENS:
            return False
        seen = self._shapes_seen.pop(key, 0) + 1              # back in at the young end
        self._shapes_seen[key] = seen
        if len(self._shapes_seen) > self.SHAPES_REMEMBERED:
            del self._shapes_seen[next(iter(self._shapes_seen))]
        return seen >= self.GRAPH_AFTER and self._room_for_a_graph()

    def _graph_step(self, entries: list[StepEntry]) -> torch.Tensor:
        graph = self._graph_for(entries)
        logits = graph.run(self, entries)
        self._graph_result = graph
        return logits

    # ------------------------------------------------------------------ requests
    def add_request(self, rid, params=None, **callbacks):
        """`add_request(rid)` makes `rid` a live request for `step()`.  `add_request(prompt_ids, GenerateParams)`
        queues a generation for `run()` instead and returns its id (a scheduler over this engine is made at the
        first such call; `token_bytes` and `on_chunk` may be passed on)."""
        if params is None:
            self.cache.add_request(rid)
            return None
        return self.scheduler.add_request(list(rid), params, **callbacks)

    @property
    def scheduler(self):
        """The scheduler behind `add_request(prompt, params)` and `run()`."""
        if self._scheduler is None:
            from .scheduler import Scheduler, SchedulerConfig
            self._scheduler = Scheduler(self, SchedulerConfig(
                max_batch_size=self.cache.max_requests, num_blocks=self.cache.num_pages,
                prefix_cache=self.cache.prefix_cache, max_num_batched_tokens=self.max_num_batched_tokens))
        return self._scheduler

    def run(self):
        """Generate for everything queued with `add_request(prompt, params)`; results by request id."""
        return self.scheduler.run()

    def end_request(self, rid) -> None:
        self.cache.release(rid)

    def has_request(self, rid) -> bool:
        return self.cache.has_request(rid)

    # ---------------------------------------------------------------------- step
    def validate(self, entries: list[StepEntry]) -> None:
        seen = set()
        vocab, limit = self.model.vocab_size, self.model.max_positions
        if not entries:
            raise ValueError("a step needs at least one entry")
        for entry in entries:
            if entry.rid in seen:
                raise ValueError(f"request {entry.rid!r} appears twice in one step")
            seen.add(entry.rid)
            if not self.cache.has_request(entry.rid):
                raise KeyError(f"request {entry.rid!r} is not live")
            if len(entry.tokens) == 0:
                raise ValueError(f"request {entry.rid!r} brings no tokens")
            if isinstance(entry.tokens, np.ndarray) or len(entry.tokens) > 64:
                # Long portions: one conversion, kept for the packing (none if the caller brings an array of ids).
                if entry.token_array is None:
                    entry.token_array = np.ascontiguousarray(entry.tokens, dtype=np.int64)
                low, high = int(entry.token_array.min()), int(entry.token_array.max())
            else:
                low, high = min(entry.tokens), max(entry.tokens)
            if not (0 <= low and high < vocab):
                raise ValueError(f"request {entry.rid!r} has a token id outside 0..{vocab - 1}")
            end = self.cache.seq_len(entry.rid) + len(entry.tokens)
            if end > limit:
                # qwen-infer/src/model.rs:896-905
                raise ValueError(f"positions up to {end} exceed max_position_embeddings {limit}")
            if any((not 0 <= int(w) < len(entry.tokens)) for w in entry.want):
                raise ValueError(f"request {entry.rid!r} wants a place outside its tokens")

    def reserve(self, entries: list[StepEntry]) -> None:
        """Pages for the new tokens of every entry, or `OutOfPages` with nothing changed for the failing one."""
        for entry in entries:
            new_len = self.cache.seq_len(entry.rid) + len(entry.tokens)
            if not self.cache.reserve(entry.rid, new_len):
                raise OutOfPages(f"no pages left for request {entry.rid!r} to reach {new_len} tokens "
                                 f"({self.cache.num_pages} pages of {self.cache.page_size})")

    def step(self, entries: list[StepEntry], reserve: bool = True) -> torch.Tensor:
        """Run the entries' tokens as one batch; float32 logits [wanted, vocab].  The step itself works on pages
        that are there: `reserve=True` (callers without a scheduler: replay, `generate`, tests) first asks the
        cache manager for the pages of the new tokens and raises `OutOfPages` if there are none;
        `reserve=False` (the scheduler, which reserves while it plans and preempts when pages run out) takes
        nothing from the pool, and an entry whose pages are missing is refused."""
        self.validate(entries)
        if reserve:
            self.reserve(entries)
        self._graph_result = None
        wanted = sum(len(entry.want) for entry in entries)
        if self._replays(entries):
            logits = self._graph_step(entries)
        else:
            ctx = build_context(entries, self.cache, self.model.device, fill=True)
            logits = self.model.decoder.forward(ctx, self.layer_caches)
        if logits.shape[0] != wanted:
            logits = logits[:wanted]        # the rows behind them belong to what the step was filled up with
        for entry in entries:
            self.cache.advance(entry.rid, self.cache.seq_len(entry.rid) + len(entry.tokens))
        self.steps += 1
        return logits
