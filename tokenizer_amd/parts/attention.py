"""Grouped-query attention over the paged cache."""
from __future__ import annotations

import math

import torch

from .base import can_fuse_decode as _can_fuse
from .base import MIXERS, POSITIONS, Mixer, Repeatable, Runtime, repeatable_of
from .spec import CacheNeed, MixerSpec, PositionSpec, TensorSpec


@MIXERS.register("gqa_attention")
class GQAttention(Mixer):
    """q/k/v projections (optional bias), position encoding, causal attention with an optional
    window over the request's pages, output projection.

    Order of operations as qwen-infer/src/model.rs:279-328 and 397-414: keys are stored after
    the position encoding, values as projected; kv head g serves query heads g*r..(g+1)*r-1
    (model.rs:571-580); scores are scaled by 1/sqrt(d) after the product; a key is visible when
    key <= query and, with a window w, key + w >= query (model.rs:119-129).
    The three projection matrices are joined into one at load time so one product makes q, k and v.
    """
    graph_safe = True


    def __init__(self, spec: MixerSpec, tensors: dict[str, torch.Tensor], runtime: Runtime):
        self.spec, self.runtime = spec, runtime
        self.n_q, self.n_kv, self.d = spec.n_heads, spec.n_kv_heads, spec.head_dim
        self.w_qkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"],
                                tensors["v_proj.weight"]], dim=0).contiguous()
        self.b_qkv = None
        if spec.qkv_bias:
            self.b_qkv = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"],
                                    tensors["v_proj.bias"]], dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]
        self.b_o = tensors.get("o_proj.bias") if spec.out_bias else None
        self.scale = float(spec.scale) if spec.scale is not None else 1.0 / math.sqrt(self.d)
        self.window = spec.window
        position = spec.position or PositionSpec("none")
        self.position = POSITIONS.get(position.kind)(position, runtime)
        self.graph_safe = bool(getattr(self.position, "graph_safe", False))

    @staticmethod
    def tensor_specs(spec: MixerSpec) -> dict[str, TensorSpec]:
        q_out, kv_out, hidden = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim, spec.hidden_size
        out = {"q_proj.weight": TensorSpec((q_out, hidden)), "k_proj.weight": TensorSpec((kv_out, hidden)),
               "v_proj.weight": TensorSpec((kv_out, hidden)), "o_proj.weight": TensorSpec((hidden, q_out))}
        if spec.qkv_bias:
            out.update({"q_proj.bias": TensorSpec((q_out,), role="vector"),
                        "k_proj.bias": TensorSpec((kv_out,), role="vector"),
                        "v_proj.bias": TensorSpec((kv_out,), role="vector")})
        if spec.out_bias:
            out["o_proj.bias"] = TensorSpec((hidden,), role="vector")
        return out

    @staticmethod
    def cache_need(spec: MixerSpec) -> CacheNeed:
        kind = "full" if spec.window is None else "window"
        return CacheNeed(kind=kind, n_kv_heads=spec.n_kv_heads, head_dim=spec.head_dim, window=spec.window)

    def repeatable(self):
        position = repeatable_of(self.position)
        if position is None:
            return None
        return Repeatable(("gqa_attention", self.n_q, self.n_kv, self.d, self.scale, self.window, position.constants),
                          (self.w_qkv, self.b_qkv, self.w_o, self.b_o) + position.tensors)

    def forward_normed(self, residual, delta, norm, ctx, cache):
        """Decode batches of few bfloat16 rows: norm + q/k/v product + bias + rotation + cache write in one
        kernel, attention, then the output product added straight into the residual stream."""
        ops = self.runtime.ops
        # The norm and the position encoding say themselves whether they have the form the fused kernels compute.
        fold = norm.fold() if delta is None else None
        behind = self.position.epilogue() if fold is not None else None
        fused = (behind is not None and self.d % 32 == 0 and cache.group is not None
                 and _can_fuse(ops, residual, self.runtime.dtype))
        if not fused:
            # The output is handed on as a delta: an output product whose K is cut over workgroups may stay in
            # parts, and the norm that takes it next adds them in its own kernel.
            return self._run(norm.apply(residual, delta), ctx, cache, pending=getattr(ops, "takes_pending", False))
        if getattr(ops, "fold_norm", lambda hidden: True)(residual.shape[1]):
            rows, norm_weight = residual, fold.weight
        else:                       # a wide model: the norm's own kernel once, not again in every workgroup
            rows, norm_weight = norm.apply(residual, None), None
        q = ops.fused_norm_qkv_rope(rows, norm_weight, fold.eps, self.w_qkv, self.b_qkv, ctx.positions,
                                    behind.cos_sin, ctx.slots[cache.group] if cache.writes else None,
                                    cache.k_pages, cache.v_pages, self.n_q, self.n_kv, self.d)
        mixed = torch.empty((q.shape[0], self.n_q * self.d), dtype=q.dtype, device=q.device)
        ops.paged_attention(q, mixed, cache.k_pages, cache.v_pages, ctx.positions, ctx.entry_of_token,
                            ctx.block_tables[cache.group], self.n_q, self.n_kv, self.d, self.window,
                            self.scale, max_position=ctx.max_position, batch=ctx)
        ops.linear_add(mixed, self.w_o, self.b_o, residual)
        return None

    def forward(self, x, ctx, cache):
        return self._run(x, ctx, cache, pending=False)

    def _run(self, x, ctx, cache, pending: bool):
        ops = self.runtime.ops
        can = getattr(ops, "can_rope_store", None)
        behind = None
        if can and can(x.shape[0], self.runtime.dtype, self.w_qkv.numel()) and self.d % 32 == 0 and cache.group is not None:
            behind = self.position.epilogue()
        if behind is not None:
            # A few dozen rows: bias, rotation and the cache write ride in the projection's epilogue.
            qkv = ops.fused_norm_qkv_rope(x, None, 0.0, self.w_qkv, self.b_qkv, ctx.positions, behind.cos_sin,
                                          ctx.slots[cache.group] if cache.writes else None, cache.k_pages,
                                          cache.v_pages, self.n_q, self.n_kv, self.d)
        else:
            qkv = ops.linear(x, self.w_qkv, self.b_qkv)   # bias joins the float accumulator
            self.position.encode_and_store(qkv, None, self.n_q, self.n_kv, self.d, ctx, cache)
        mixed = torch.empty((x.shape[0], self.n_q * self.d), dtype=x.dtype, device=x.device)
        ops.paged_attention(qkv, mixed, cache.k_pages, cache.v_pages, ctx.positions, ctx.entry_of_token,
                            ctx.block_tables[cache.group], self.n_q, self.n_kv, self.d, self.window,
                            self.scale, max_position=ctx.max_position, batch=ctx)
        return ops.linear(mixed, self.w_o, self.b_o, pending=True) if pending else ops.linear(mixed, self.w_o, self.b_o)
