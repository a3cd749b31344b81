"""The engine: a model, its cache and the one step function everything else is built on."""
from __future__ import annotations

import torch

from ..cache import CacheManager, CachePools, OutOfPages
from ..config import load_config
from ..config.base import ModelConfig
from ..config.registry import get_architecture
from ..parts import DecoderModel, LayerCache, Runtime, cache_needs, expected_tensors
from ..weights import load_weights, random_tensors, stored_form
from .batch import StepContext, StepEntry, build_context

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
        self.decoder = DecoderModel(self.spec, tensors, self.runtime)
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


class Engine:
    """Owns the cache of one model and runs steps.

    `step(entries)` runs exactly the tokens it is given, as one batch, against what earlier steps
    left in the cache, and returns float32 logits at the wanted places, in the order of the
    entries and of each entry's `want`.
    """

    def __init__(self, model: Model, num_pages: int | None = None, page_size: int = 16, max_requests: int = 8,
                 max_tokens: int | None = None, prefix_cache: bool = False):
        if num_pages is None:
            if max_tokens is None:
                raise ValueError("give num_pages or max_tokens")
            num_pages = -(-max_tokens // page_size)
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

    @property
    def max_positions(self) -> int:
        return self.model.max_positions

    # ------------------------------------------------------------------- sampling
    def argmax(self, logits: torch.Tensor, rows: list[int] | None = None) -> list[int]:
        """Greedy ids of the given rows of a step's logits, picked on the device."""
        picked = self.model.runtime.ops.argmax(logits).cpu().tolist()
        return picked if rows is None else [picked[row] for row in rows]

    def rows_to_host(self, logits: torch.Tensor, rows: list[int]):
        return logits[rows].float().cpu().numpy()

    # ------------------------------------------------------------------ requests
    def add_request(self, rid) -> None:
        self.cache.add_request(rid)

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
            if not entry.tokens:
                raise ValueError(f"request {entry.rid!r} brings no tokens")
            if any((not 0 <= int(t) < vocab) for t in entry.tokens):
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

    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        self.validate(entries)
        self.reserve(entries)
        ctx = build_context(entries, self.cache, self.model.device)
        logits = self.model.decoder.forward(ctx, self.layer_caches)
        for entry in entries:
            self.cache.advance(entry.rid, self.cache.seq_len(entry.rid) + len(entry.tokens))
        self.steps += 1
        return logits
