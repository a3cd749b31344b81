"""RMSNorm over the last axis, fused with the residual add that precedes it."""
from __future__ import annotations

import torch

from .base import NORMS, Norm, NormFold, Repeatable, Runtime
from .spec import NormSpec, TensorSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    """y = x / sqrt(mean(x^2) + eps) * weight (qwen-infer/src/model.rs:594-599), in float32."""
    graph_safe = True


    def __init__(self, spec: NormSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.size, self.eps = spec.size, float(spec.eps)
        self.weight = tensors["weight"]
        self.runtime = runtime

    @staticmethod
    def tensor_specs(spec: NormSpec) -> dict[str, TensorSpec]:
        return {"weight": TensorSpec((spec.size,), init="ones", role="vector")}

    def fold(self):
        return NormFold(self.weight, self.eps)

    def repeatable(self):
        return Repeatable(("rmsnorm", self.size, self.eps), (self.weight,))

    def apply(self, residual, delta, rows=None):
        n_rows = residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n_rows, self.size), dtype=self.runtime.dtype, device=residual.device)
        return self.runtime.ops.add_rmsnorm(residual, delta, self.weight, self.eps, out, rows,
                                            store_residual=rows is None)
