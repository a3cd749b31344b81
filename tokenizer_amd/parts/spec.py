"""Descriptions of a model as data: parts, layers and the order they run in.

An architecture turns its configuration into a `ModelSpec`.  Nothing below
knows any architecture: every size and constant is a field, every part is named
by a `kind` that the part registries resolve, and the run order is a list of
`ScheduleEntry`, which may name a layer twice or point a layer at another
layer's cache.
"""
from __future__ import annotations

import dataclasses
from typing import Any


@dataclasses.dataclass(frozen=True)
class TensorSpec:
    """One tensor a part needs from the weight file.

    `init` says how the random-weights mode fills it: "normal" (N(0, std)),
    "ones" or "zeros".  `role` says how it is kept in memory: "matrix" tensors
    feed matrix products and are held in the compute dtype, "vector" tensors
    (norm scales, biases) are small and held in float32, "table" tensors are
    integer tables kept as int32, "keep" tensors stay as the file stores them.
    """
    shape: tuple[int, ...]
    init: str = "normal"
    std: float = 0.02
    role: str = "matrix"


@dataclasses.dataclass(frozen=True)
class CacheNeed:
    """What a mixer asks of the cache manager for one layer.

    kind "full": keys and values of every position, in pages.
    kind "window": only the last `window` + 1 positions are ever read; pages
    wholly behind the window are given back.
    kind "none": no pages.
    `state_shape`: per-request state of fixed size kept in a slot, or None.
    """
    kind: str = "none"
    n_kv_heads: int = 0
    head_dim: int = 0
    window: int | None = None
    state_shape: tuple[int, ...] | None = None
    state_dtype: str = "float32"

    def page_key(self) -> tuple:
        """Layers with equal keys share one group of pages and one block table."""
        return (self.kind, self.n_kv_heads, self.head_dim, self.window)


@dataclasses.dataclass(frozen=True)
class NormSpec:
    kind: str
    size: int
    eps: float
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)


@dataclasses.dataclass(frozen=True)
class PositionSpec:
    """Position encoding applied to queries and keys inside a mixer."""
    kind: str                     # "rope_half_split", "none", ...
    head_dim: int = 0
    theta: float = 0.0
    max_positions: int = 0
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)


@dataclasses.dataclass(frozen=True)
class MixerSpec:
    kind: str                     # "gqa_attention", ...
    hidden_size: int
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    qkv_bias: bool = False
    out_bias: bool = False
    window: int | None = None
    scale: float | None = None    # None = 1/sqrt(head_dim)
    position: PositionSpec | None = None
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)


@dataclasses.dataclass(frozen=True)
class FeedForwardSpec:
    kind: str                     # "gated_dense", ...
    hidden_size: int
    intermediate_size: int = 0
    activation: str = "silu"
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    """One layer: which block arrangement, which parts, and their tensor name prefixes.

    Either sub-layer may be absent (None for the part and for its norm; at least one is there): a layer of a
    mixer alone, or of a feed-forward alone.  Since the schedule is a list of layers, any chain of sub-layers
    (two mixers before one feed-forward, say) is a run of such layers.
    """
    block: str                    # "pre_norm", ...
    mixer: MixerSpec | None
    feed_forward: FeedForwardSpec | None
    mixer_norm: NormSpec | None
    feed_forward_norm: NormSpec | None
    mixer_prefix: str = ""
    feed_forward_prefix: str = ""
    mixer_norm_prefix: str = ""
    feed_forward_norm_prefix: str = ""

    def __post_init__(self):
        if self.mixer is None and self.feed_forward is None:
            raise ValueError("a layer needs a mixer or a feed-forward")
        for part, norm, what in ((self.mixer, self.mixer_norm, "mixer"),
                                 (self.feed_forward, self.feed_forward_norm, "feed-forward")):
            if (part is None) != (norm is None):
                raise ValueError(f"a layer's {what} and its norm are there together or not at all")


@dataclasses.dataclass(frozen=True)
class ScheduleEntry:
    """Run `layer`; its mixer uses the cache of `cache_of` (default: its own).

    A layer that reads another layer's cache writes nothing into it.
    """
    layer: int
    cache_of: int | None = None


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding_name: str
    layers: tuple[LayerSpec, ...]
    schedule: tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    final_norm_prefix: str
    tied_head: bool
    head_name: str                # used when the head is not tied
    embedding_std: float = 0.02
    frame: str = "decoder"        # what stands around the layers (`parts.base.FRAMES`)
    options: dict[str, Any] = dataclasses.field(default_factory=dict, hash=False, compare=False)   # the frame's own constants
