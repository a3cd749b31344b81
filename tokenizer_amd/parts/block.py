"""Arrangements of norms, mixer and feed-forward around the residual stream."""
from __future__ import annotations

from .base import BLOCKS, Block, Repeatable, repeatable_of


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    """x + mixer(norm1(x)), then + feed_forward(norm2(.)) (qwen-infer/src/model.rs:615-622).

    The residual stream is float32.  Each sub-layer's output is handed on as a pending `delta`
    so that the add fuses into the next norm; a part that added its output itself hands on None.
    A sub-layer that the layer does not have (None) is passed over.
    """
    graph_safe = True


    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward

    def repeatable(self, cache):
        """The layer's library calls depend on its four parts and on which pages it reads and writes."""
        parts = [repeatable_of(part) for part in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward)]
        if any(part is None for part in parts) or cache.state is not None:
            return None
        return Repeatable(("pre_norm", cache.group, cache.writes) + tuple(part.constants for part in parts),
                          sum((part.tensors for part in parts), ()) + (cache.k_pages, cache.v_pages))

    def forward(self, residual, delta, ctx, cache):
        if self.mixer is not None:
            delta = self.mixer.forward_normed(residual, delta, self.mixer_norm, ctx, cache)
        if self.feed_forward is not None:
            delta = self.feed_forward.forward_normed(residual, delta, self.feed_forward_norm, ctx)
        return delta
