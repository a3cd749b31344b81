"""Interfaces of the parts a layer is put together from, and their registries.

A part is built from its spec, the tensors it asked for and a `Runtime`
(compute dtype, device, kernel library).  No part knows which model it is in.

Interfaces
----------
Norm            tensor_specs(spec) -> {local name: TensorSpec}
                apply(residual, delta, rows=None) -> normalised rows in the compute dtype.
                Optional: fold() -> NormFold, if the norm is x / sqrt(mean(x^2) + eps) * weight for some weight:
                a mixer or feed-forward may then take it into the prologue of its own product.
                `residual` is the float32 stream [T, H]; `delta` (or None) is added to it first and,
                unless `rows` picks a subset, the sum is stored back.  `delta` may also be a product still
                in parts (`kernels.PendingSum`, which the kernel library's `add_rmsnorm` takes as it is): a
                norm with kernels of its own calls `as_tensor(delta)` first.
PositionEncoding
                encode_and_store(qkv, geometry, ctx, cache, bias): adds the projection bias, encodes
                the query and key heads in place and writes keys and values of this step into `cache`.
                Optional: epilogue() -> StoreEpilogue, if the encoding is a rotation of half-split pairs by a
                table (or nothing at all): the fused projection then does it, and the store, in its epilogue.
Mixer           tensor_specs(spec), cache_need(spec) -> CacheNeed
                forward(x [T, H], ctx: StepContext, cache: LayerCache) -> [T, H] in the compute dtype.
                Optional: forward_normed(residual, delta, norm, ctx, cache) to fold the norm before it and the
                residual add after it into its own kernels (returns None when it added its output itself; what
                it returns is only ever handed to a norm as its delta, so it may be a product still in parts).
FeedForward     tensor_specs(spec); forward(x [T, H], ctx) -> [T, H]; optional forward_normed likewise.
Block           arranges two norms, a mixer and a feed-forward around the residual stream (either sub-layer may
                be absent: None for the part and its norm):
                forward(residual, delta, ctx, cache) -> delta still to be added.

Frame           what stands around the layers: `ModelSpec.frame` names it.  Static `expected_tensors(spec)` (every
                tensor name the model reads, with its `TensorSpec`) and `cache_needs(spec)` (one `CacheNeed` per
                layer); built from (spec, tensors, runtime); `graph_safe`; `forward(ctx, layer_caches)` -> float32
                logits [wanted, vocab].  The built-in "decoder" frame (`parts.model.DecoderModel`) is embedding,
                layers in schedule order, final norm, head, with `embed(ctx)` and `logits(residual, delta, ctx)` as
                the two places a subclass changes (a scaled embedding, a learned position table, a head bias, a cap
                on the logits); its constants beyond the spec's fields travel in `ModelSpec.options`.

Every part may also say `repeatable() -> Repeatable` (a block: `repeatable(cache)`): that on the device its forward
does nothing but call the kernel library, and that those calls depend on the part only through the constants and the
tensors it lists.  The model then records the calls of one such layer on a step's batch and makes them again for
the like layers after it, with their tensors' addresses put in place (`kernels.LaunchTape`), instead of running
their Python.  The promise is the class's own: a subclass does not inherit it and has to give it again.
"""
from __future__ import annotations

import dataclasses
from typing import Any

import torch

from .spec import CacheNeed, TensorSpec


@dataclasses.dataclass
class Runtime:
    dtype: torch.dtype
    device: torch.device
    ops: Any                      # tokenizer_amd.kernels.Ops (or a stand-in with the same methods)


class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: dict[str, type] = {}

    def register(self, kind: str, cls: type | None = None, replace: bool = False):
        def put(target: type) -> type:
            if kind in self._items and not replace:
                raise ValueError(f"{self.what} {kind!r} is already registered")
            self._items[kind] = target
            return target
        return put if cls is None else put(cls)

    def get(self, kind: str) -> type:
        try:
            return self._items[kind]
        except KeyError:
            raise KeyError(f"unknown {self.what} {kind!r}; registered: {', '.join(sorted(self._items))}") from None

    def kinds(self) -> list[str]:
        return sorted(self._items)


NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
BLOCKS = Registry("block")
FRAMES = Registry("model frame")


class Part:
    """Common base: a part names its tensors and is built from them.

    `graph_safe` says that the part's forward only launches device work whose shape depends on the
    batch's sizes, never on host-side values of the batch (positions, request ids): only then may a
    decode step be captured once and replayed.  Parts are taken not to be unless they say so.
    """
    graph_safe = False

    @staticmethod
    def tensor_specs(spec) -> dict[str, TensorSpec]:
        return {}


@dataclasses.dataclass
class NormFold:
    """A norm in the form the fused products take into their prologue: y = x / sqrt(mean(x^2) + eps) * weight,
    with `weight` float32 [H] on the device.  A norm of that form says so through `Norm.fold()`, whatever its
    class and however it derives the weight from its tensors."""
    weight: torch.Tensor
    eps: float


@dataclasses.dataclass
class StoreEpilogue:
    """What the fused q/k/v projection can do behind its bias: rotate the half-split pairs of every query and
    key head by the row of `cos_sin` (float32 [positions, d]: cos half, then sin half) at the token's position,
    `cos_sin` None meaning no rotation, and write keys and values into their pages.  A position encoding that is
    of that form says so through `PositionEncoding.epilogue()`."""
    cos_sin: torch.Tensor | None


@dataclasses.dataclass(frozen=True)
class Repeatable:
    """What a part's library calls depend on: `constants` (hashable; parts whose constants are equal make the same
    calls) and `tensors` (their addresses are what differs from one such part to the next; None where a part has
    none, the same places in every like part)."""
    constants: tuple
    tensors: tuple


def repeatable_of(part, *args) -> Repeatable | None:
    """The part's `repeatable(*args)` if its own class gives that promise, else None."""
    if part is None:
        return Repeatable(("absent",), ())
    if "repeatable" not in vars(type(part)):
        return None
    return part.repeatable(*args)


class Norm(Part):
    def apply(self, residual: torch.Tensor, delta: torch.Tensor | None,
              rows: torch.Tensor | None = None) -> torch.Tensor:
        raise NotImplementedError

    def fold(self) -> NormFold | None:
        """The norm as a product's prologue can compute it, or None (the parts then call `apply`)."""
        return None


class PositionEncoding(Part):
    def encode_and_store(self, qkv, bias, n_q: int, n_kv: int, head_dim: int, ctx, cache) -> None:
        raise NotImplementedError

    def epilogue(self) -> StoreEpilogue | None:
        """The encoding as the fused projection's epilogue can apply it, or None (`encode_and_store` is called)."""
        return None


class Mixer(Part):
    @staticmethod
    def cache_need(spec) -> CacheNeed:
        return CacheNeed()

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        raise NotImplementedError

    def forward_normed(self, residual, delta, norm: Norm, ctx, cache):
        """The sub-layer from the residual stream on: add `delta`, normalise, mix.  Returns the output still
        to be added to the stream, or None if the part added it itself.  A part may override this to fold
        the norm and the add into its own kernels; this default keeps them apart."""
        return self.forward(norm.apply(residual, delta), ctx, cache)


class FeedForward(Part):
    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError

    def forward_normed(self, residual, delta, norm: Norm, ctx):
        """As `Mixer.forward_normed`, for the feed-forward."""
        return self.forward(norm.apply(residual, delta), ctx)


class Block:
    graph_safe = False

    def forward(self, residual: torch.Tensor, delta: torch.Tensor | None, ctx, cache) -> torch.Tensor:
        raise NotImplementedError


def as_tensor(delta):
    """The delta as a tensor: a product still in parts has them added now."""
    resolve = getattr(delta, "resolve", None)
    return resolve() if resolve is not None and not isinstance(delta, torch.Tensor) else delta


def can_fuse_decode(ops, residual, dtype) -> bool:
    """Whether the kernel library offers its fused decode products for these rows of the residual stream
    (few bfloat16 rows of a width whose normalised copy fits in LDS); a library without them says no."""
    check = getattr(ops, "can_fuse_decode", None)
    return bool(check and check(residual.shape[0], dtype, residual.shape[1]))
