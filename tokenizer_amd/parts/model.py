"""A decoder put together from a `ModelSpec`: embedding, layers in schedule order, final norm, head."""
from __future__ import annotations

import dataclasses

import torch

from .base import BLOCKS, FEED_FORWARDS, FRAMES, MIXERS, NORMS, Runtime, repeatable_of
from .spec import CacheNeed, ModelSpec, TensorSpec


def _prefixed(prefix: str, specs: dict[str, TensorSpec]) -> dict[str, TensorSpec]:
    return {f"{prefix}.{name}" if prefix else name: spec for name, spec in specs.items()}


def expected_tensors(spec: ModelSpec) -> dict[str, TensorSpec]:
    """Every tensor name the model reads from the weight file, with its shape: its frame says."""
    return FRAMES.get(spec.frame).expected_tensors(spec)


def cache_needs(spec: ModelSpec) -> list[CacheNeed]:
    """What each layer asks of the cache manager, by layer index: the model's frame says."""
    return FRAMES.get(spec.frame).cache_needs(spec)


def build_model(spec: ModelSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
    """The model of `spec` in the frame it names."""
    return FRAMES.get(spec.frame)(spec, tensors, runtime)


def _strip(prefix: str, tensors: dict[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    lead = prefix + "."
    return {name[len(lead):]: value for name, value in tensors.items() if name.startswith(lead)}


@dataclasses.dataclass
class LayerCache:
    """What one scheduled layer may touch of the cache in a step."""
    group: int | None = None                # index into ctx.block_tables / ctx.slots
    k_pages: torch.Tensor | None = None     # [n_pages, n_kv, page_size, d]
    v_pages: torch.Tensor | None = None
    state: torch.Tensor | None = None       # [n_slots, *state_shape]
    writes: bool = True                     # False when the layer reads another layer's cache
    makes: dict = dataclasses.field(default_factory=dict, repr=False, compare=False)   # what the layers run on it depend on


class _Make:
    """What one scheduled layer's library calls depend on: `key` (layers with equal keys make the same calls) and the
    addresses of its tensors, in the order in which every layer of that key lists them."""

    def __init__(self, constants: tuple, tensors: tuple):
        # (Strides and alignment too: the recorded layer's tensors passed the wrappers' checks, a like layer's must
        # be laid out the same way to pass them unseen.)
        self.key = (constants, tuple(None if t is None else (tuple(t.shape), t.dtype, t.stride(), t.data_ptr() % 16)
                                     for t in tensors))
        self.addresses = tuple(0 if t is None else t.data_ptr() for t in tensors)
        self.tensors = tensors                 # kept, so the addresses stay theirs
        # The address maps from recorded layers of the same key to this one, by the recorded layer's make itself
        # (never by its id, which another object may get once that make is gone): they live and die with the
        # makes, which belong to one engine's cache entries.
        self.puts: dict["_Make", object] = {}
        self.held: frozenset = frozenset()     # addresses of every tensor the layer's parts hold, listed or not


@dataclasses.dataclass
class _Recorded:
    """One layer's library calls on this step's batch, with what they were recorded for."""
    tape: object                  # kernels.LaunchTape
    make: _Make
    coming: tuple                 # the addresses of what the layer was handed
    result: object                # what it handed on (its buffers serve every layer that repeats the calls)
    unlisted: frozenset = frozenset()   # addresses on the tape of tensors the layer holds without having listed them


def _tensor_addresses(part, seen=None) -> set:
    """The addresses of every tensor that a part holds as an attribute, itself or through the parts it holds (a
    block's norms, a mixer's position encoding), lists and tuples included."""
    seen = set() if seen is None else seen
    found: set[int] = set()
    if part is None or id(part) in seen or not hasattr(part, "__dict__"):
        return found
    seen.add(id(part))
    for value in vars(part).values():
        for item in (value if isinstance(value, (list, tuple)) else (value,)):
            if isinstance(item, torch.Tensor):
                if item.numel():
                    found.add(item.data_ptr())
            elif hasattr(item, "__dict__") and not isinstance(item, (type, Runtime)) \
                    and type(item).__module__.split(".")[0] not in ("torch", "ctypes", "threading", "builtins"):
                found |= _tensor_addresses(item, seen)
    return found


def _coming(delta):
    """What a layer is handed besides the stream: (a word for its form, the addresses a library call would be given).
    Forms this module does not know make the layer run on its own."""
    if delta is None:
        return "none", ()
    if isinstance(delta, torch.Tensor):
        return ("tensor", tuple(delta.shape), delta.dtype, delta.is_contiguous()), (delta.data_ptr(),)
    partial, bias = getattr(delta, "partial", None), getattr(delta, "bias", None)
    if isinstance(partial, torch.Tensor) and bias is None:
        return ("parts", tuple(partial.shape), getattr(delta, "dtype", None)), (partial.data_ptr(),)
    return None, ()


def _addresses_put(recorded: tuple, wanted: tuple):
    """The map from the recorded layer's addresses to another layer's, or False if one address would have to stand
    for two."""
    put: dict[int, int] = {}
    for a, b in zip(recorded, wanted):
        if put.setdefault(a, b) != b:
            return False
    return {a: b for a, b in put.items() if a != b}


@FRAMES.register("decoder")
class DecoderModel:
    """Weights and parts of one model: embedding, layers in schedule order, final norm, head.  It owns no cache:
    `forward` is handed the step's context (token ids, positions, block tables) and one `LayerCache` per schedule
    entry.  A frame that differs only before the first layer or behind the last overrides `embed` or `logits`
    (and `expected_tensors`, if it reads tensors of its own)."""

    @staticmethod
    def expected_tensors(spec: ModelSpec) -> dict[str, TensorSpec]:
        out = {spec.embedding_name: TensorSpec((spec.vocab_size, spec.hidden_size), std=spec.embedding_std)}
        for layer in spec.layers:
            if layer.mixer is not None:
                out.update(_prefixed(layer.mixer_norm_prefix, NORMS.get(layer.mixer_norm.kind).tensor_specs(layer.mixer_norm)))
                out.update(_prefixed(layer.mixer_prefix, MIXERS.get(layer.mixer.kind).tensor_specs(layer.mixer)))
            if layer.feed_forward is not None:
                out.update(_prefixed(layer.feed_forward_norm_prefix,
                                     NORMS.get(layer.feed_forward_norm.kind).tensor_specs(layer.feed_forward_norm)))
                out.update(_prefixed(layer.feed_forward_prefix,
                                     FEED_FORWARDS.get(layer.feed_forward.kind).tensor_specs(layer.feed_forward)))
        out.update(_prefixed(spec.final_norm_prefix, NORMS.get(spec.final_norm.kind).tensor_specs(spec.final_norm)))
        if not spec.tied_head:
            out[spec.head_name] = TensorSpec((spec.vocab_size, spec.hidden_size))
        return out

    @staticmethod
    def cache_needs(spec: ModelSpec) -> list[CacheNeed]:
        """(A layer without a mixer asks for nothing.)"""
        return [MIXERS.get(layer.mixer.kind).cache_need(layer.mixer) if layer.mixer is not None else CacheNeed()
                for layer in spec.layers]

    def __init__(self, spec: ModelSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.spec, self.runtime = spec, runtime
        self.embedding = tensors[spec.embedding_name]
        self.blocks = []
        for layer in spec.layers:
            mixer_norm = mixer = ff_norm = feed_forward = None
            if layer.mixer is not None:
                mixer_norm = NORMS.get(layer.mixer_norm.kind)(layer.mixer_norm, _strip(layer.mixer_norm_prefix, tensors), runtime)
                mixer = MIXERS.get(layer.mixer.kind)(layer.mixer, _strip(layer.mixer_prefix, tensors), runtime)
            if layer.feed_forward is not None:
                ff_norm = NORMS.get(layer.feed_forward_norm.kind)(layer.feed_forward_norm,
                                                                  _strip(layer.feed_forward_norm_prefix, tensors), runtime)
                feed_forward = FEED_FORWARDS.get(layer.feed_forward.kind)(layer.feed_forward,
                                                                         _strip(layer.feed_forward_prefix, tensors), runtime)
            self.blocks.append(BLOCKS.get(layer.block)(mixer_norm, mixer, ff_norm, feed_forward))
        self.final_norm = NORMS.get(spec.final_norm.kind)(spec.final_norm, _strip(spec.final_norm_prefix, tensors), runtime)
        self.head = self.embedding if spec.tied_head else tensors[spec.head_name]
        parts = [self.final_norm] + [p for b in self.blocks if hasattr(b, "mixer")
                                     for p in (b, b.mixer_norm, b.mixer, b.feed_forward_norm, b.feed_forward)
                                     if p is not None]
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in parts) and \
            all(hasattr(b, "mixer") for b in self.blocks)
        self.repeat_layers = True      # record one layer's library calls and make them again for the like ones
        self.layers_repeated = 0       # how many scheduled layers have run that way so far
        self.promises_broken = 0       # recordings thrown away because a call took a tensor the parts had not listed

    def _make_of(self, block, layer: int, cache: "LayerCache"):
        """The make of a scheduled layer on this cache, or None if the block does not promise to be repeatable.
        Worked out once and kept on the cache entry."""
        if layer not in cache.makes:
            said = repeatable_of(block, cache)
            make = None if said is None else _Make(said.constants, said.tensors)
            if make is not None:
                make.held = frozenset(_tensor_addresses(block))
            cache.makes[layer] = make
        return cache.makes[layer]

    def embed(self, ctx) -> torch.Tensor:
        """The float32 residual stream [tokens, hidden] the first layer starts from."""
        residual = torch.empty((ctx.n_tokens, self.spec.hidden_size), dtype=torch.float32, device=self.runtime.device)
        return self.runtime.ops.embedding(ctx.token_ids, self.embedding, residual)

    def logits(self, residual: torch.Tensor, delta, ctx) -> torch.Tensor:
        """Float32 logits at the wanted rows from the stream and what is still to be added to it.  Only the wanted
        rows are normalised and multiplied with the head (the reference keeps the last row,
        qwen-infer/src/model.rs:1224-1242)."""
        wanted = self.final_norm.apply(residual, delta, rows=ctx.want_rows)
        return self.runtime.ops.linear(wanted, self.head, out_dtype=torch.float32)

    def forward(self, ctx, layer_caches: list[LayerCache]) -> torch.Tensor:
        """Run the tokens of `ctx` through the schedule; float32 logits [len(want_rows), vocab]."""
        ops = self.runtime.ops
        residual = self.embed(ctx)
        delta = None
        # Like layers make the same library calls on a batch: the calls of the first are recorded and made again
        # for the others with their tensors' addresses put in place, which spares those layers' Python (about
        # two thirds of an eager step's host time; a step of a small model is bound by it).  Not while a graph
        # is recorded or warmed up: that happens once, and the library times its products there.
        record = getattr(ops, "record_launches", None) if self.repeat_layers and not getattr(ops, "capturing", False) else None
        tapes: dict = {}
        for entry, cache in zip(self.spec.schedule, layer_caches):
            block = self.blocks[entry.layer]
            make = self._make_of(block, entry.layer, cache) if record is not None else None
            form, addresses = _coming(delta) if make is not None else (None, ())
            if form is None:
                delta = block.forward(residual, delta, ctx, cache)
                continue
            recorded = tapes.get((make.key, form))
            if recorded is None:
                with record() as tape:
                    out = block.forward(residual, delta, ctx, cache)
                if _coming(out)[0] == form:       # what it hands on looks like what it was handed: it can follow itself
                    # The promise is checked as far as the host can see: a call that took a tensor which the
                    # layer's parts hold but did not list depends on the layer through more than the list.
                    unlisted = (make.held - set(make.addresses)) & tape.addresses()
                    tapes[(make.key, form)] = _Recorded(tape, make, addresses, out, frozenset(unlisted))
                delta = out
                continue
            put = make.puts.get(recorded.make)
            if put is None:
                if recorded.unlisted <= make.held:     # (a tensor that both layers hold, a shared table, is the same one)
                    put = _addresses_put(recorded.make.addresses, make.addresses)
                else:
                    put, self.promises_broken = False, self.promises_broken + 1
                make.puts[recorded.make] = put
            if put is False:                      # no single map (one tensor in two places there, two here), or a broken promise
                delta = block.forward(residual, delta, ctx, cache)
                continue
            if addresses != recorded.coming:
                put = dict(put)
                put.update(zip(recorded.coming, addresses))
            recorded.tape.replay(put)
            self.layers_repeated += 1
            delta = recorded.result               # the recorded layer's buffers hold this layer's output now
        if ctx.want_rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.runtime.device)
        return self.logits(residual, delta, ctx)
