"""Position encodings applied to queries and keys before the keys go into the cache."""
from __future__ import annotations

import torch

from .base import POSITIONS, PositionEncoding, Repeatable, Runtime, StoreEpilogue
from .spec import PositionSpec


@POSITIONS.register("none")
class NoPosition(PositionEncoding):
    """No encoding: the projection bias is added and keys and values are stored as they are."""
    graph_safe = True


    def __init__(self, spec: PositionSpec, runtime: Runtime):
        self.runtime = runtime

    def table(self):
        return None

    def repeatable(self):
        return Repeatable(("none",), ())

    def epilogue(self):
        # A subclass that encodes in its own way inherits this method but not the promise: it has to offer an
        # epilogue of its own (or none).
        if type(self).encode_and_store is not NoPosition.encode_and_store:
            return None
        return StoreEpilogue(self.table())

    def encode_and_store(self, qkv, bias, n_q, n_kv, head_dim, ctx, cache):
        slots = ctx.slots[cache.group] if cache.writes else None
        self.runtime.ops.rope_store(qkv, bias, ctx.positions, self.table(), slots,
                                    cache.k_pages if cache.writes else None,
                                    cache.v_pages if cache.writes else None, n_q, n_kv, head_dim)


@POSITIONS.register("rope_half_split")
class RotaryHalfSplit(NoPosition):
    """Rotation of the two halves of a head against each other (qwen-infer/src/model.rs:131-172).

    inv_freq[i] = 1 / theta^(2i/d) is computed in float64 and kept as float32; the angle of
    position p is p * inv_freq[i] in float32; the table holds cos then sin of the d/2 angles for
    every position up to `max_positions`.  Keys are stored after the rotation.
    """

    _tables: dict[tuple, torch.Tensor] = {}

    def __init__(self, spec: PositionSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        if spec.head_dim % 2:
            raise ValueError(f"rope needs an even head size, found {spec.head_dim}")
        d = spec.head_dim
        key = (d, float(spec.theta), spec.max_positions, str(runtime.device))
        if key not in self._tables:               # the layers of a model share one table
            inv_freq = torch.tensor([1.0 / (float(spec.theta) ** (i / d)) for i in range(0, d, 2)],
                                    dtype=torch.float64).to(torch.float32)
            positions = torch.arange(spec.max_positions, dtype=torch.float32)
            angles = positions[:, None] * inv_freq[None, :]
            self._tables[key] = torch.cat([angles.cos(), angles.sin()], dim=1).contiguous().to(runtime.device)
        self.cos_sin = self._tables[key]
        self.max_positions = spec.max_positions

    def table(self):
        return self.cos_sin

    def repeatable(self):
        return Repeatable(("rope_half_split", self.max_positions), (self.cos_sin,))
