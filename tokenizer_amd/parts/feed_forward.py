"""Dense gated feed-forward."""
from __future__ import annotations

import torch

from .base import can_fuse_decode as _can_fuse
from .base import FEED_FORWARDS, FeedForward, Repeatable, Runtime
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
        gate, up, down = tensors["gate_proj.weight"], tensors["up_proj.weight"], tensors["down_proj.weight"]
        # The bfloat16 products read eight elements of K at a time.  An inner width that is no multiple of
        # eight is filled up with zero rows of gate and up and zero columns of down: act(0) * 0 = 0 meets a
        # zero weight, so every sum keeps its terms and gains only zeros.
        fill = (-spec.intermediate_size) % 8 if runtime.dtype == torch.bfloat16 else 0
        if fill:
            rows = gate.new_zeros((fill, gate.shape[1]))
            gate, up = torch.cat([gate, rows], dim=0), torch.cat([up, rows], dim=0)
            down = torch.cat([down, down.new_zeros((down.shape[0], fill))], dim=1).contiguous()
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = down

    @staticmethod
    def tensor_specs(spec: FeedForwardSpec) -> dict[str, TensorSpec]:
        return {"gate_proj.weight": TensorSpec((spec.intermediate_size, spec.hidden_size)),
                "up_proj.weight": TensorSpec((spec.intermediate_size, spec.hidden_size)),
                "down_proj.weight": TensorSpec((spec.hidden_size, spec.intermediate_size))}

    def repeatable(self):
        return Repeatable(("gated_dense",), (self.w_gate_up, self.w_down))

    def forward_normed(self, residual, delta, norm, ctx):
        """Decode batches of few bfloat16 rows: norm + gate/up product + activation in one kernel, then the
        down product added straight into the residual stream."""
        ops = self.runtime.ops
        fold = norm.fold() if delta is None else None      # the norm says whether it has the form the kernel computes
        if fold is None or not _can_fuse(ops, residual, self.runtime.dtype):
            # The output is handed on as a delta: a down product whose K is cut over workgroups may stay in
            # parts, and the norm that takes it next adds them in its own kernel.
            return self._run(norm.apply(residual, delta), pending=getattr(ops, "takes_pending", False))
        if getattr(ops, "fold_norm", lambda hidden: True)(residual.shape[1]):
            act = ops.fused_norm_gated(residual, fold.weight, fold.eps, self.w_gate_up)
        else:                       # a wide model: the norm's own kernel once, not again in every workgroup
            act = ops.fused_norm_gated(norm.apply(residual, None), None, fold.eps, self.w_gate_up)
        ops.linear_add(act, self.w_down, None, residual)
        return None

    def forward(self, x, ctx):
        return self._run(x, pending=False)

    def _run(self, x, pending: bool):
        ops = self.runtime.ops
        act = ops.linear_silu_gate(x, self.w_gate_up)
        return ops.linear(act, self.w_down, pending=True) if pending else ops.linear(act, self.w_down)
