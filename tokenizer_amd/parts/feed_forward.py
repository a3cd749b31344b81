"""Dense gated feed-forward."""
from __future__ import annotations

import torch

from .base import FEED_FORWARDS, FeedForward, Runtime
from .spec import FeedForwardSpec, TensorSpec


@FEED_FORWARDS.register("gated_dense")
class GatedDense(FeedForward):
    """down(act(gate(x)) * up(x)) without biases (qwen-infer/src/model.rs:245-249).

    gate and up are joined into one matrix at load time; the activation and the product with
    `up` run in float32 in one kernel.
    """
    graph_safe = True


    def __init__(self, spec: FeedForwardSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        if spec.activation != "silu":
            raise ValueError(f"gated_dense knows the silu activation, not {spec.activation!r}")
        self.spec, self.runtime = spec, runtime
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    @staticmethod
    def tensor_specs(spec: FeedForwardSpec) -> dict[str, TensorSpec]:
        return {"gate_proj.weight": TensorSpec((spec.intermediate_size, spec.hidden_size)),
                "up_proj.weight": TensorSpec((spec.intermediate_size, spec.hidden_size)),
                "down_proj.weight": TensorSpec((spec.hidden_size, spec.intermediate_size))}

    def forward(self, x, ctx):
        ops = self.runtime.ops
        return ops.linear(ops.linear_silu_gate(x, self.w_gate_up), self.w_down)
