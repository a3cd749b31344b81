"""Plain, slow Qwen2 decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference (paths relative to the reference
tree).  It reads a model folder with the `safetensors` package and torch on the
CPU and shares no code with `tokenizer_amd`.  Everything is computed in the
dtype given (float32 by default, float64 for a tighter oracle).
"""
from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------- io
def load_folder(folder: str, dtype=torch.float32):
    """config.json as a dict and every tensor of model.safetensors, upcast.

    qwen-infer/src/model.rs:776-786 (file is converted to f32 on read).
    """
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    tensors = {k: v.to(dtype) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, tensors


# ------------------------------------------------------------------------ parts
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w over the last axis.

    qwen-infer/src/model.rs:594-599 (candle `rms_norm(size, eps, vb)`).
    """
    mean_sq = (x * x).mean(dim=-1, keepdim=True)
    return x / torch.sqrt(mean_sq + eps) * weight


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """y = x W^T (+ b), W is [out, in].  qwen-infer/src/model.rs:268-272."""
    y = x @ weight.t()
    if bias is not None:
        y = y + bias
    return y


def rope_tables(theta: float, head_dim: int, n_positions: int, dtype=torch.float32):
    """cos, sin of shape (n_positions, head_dim/2).

    inv_freq[i] = 1 / theta^(2i/d) in f64, stored in the working dtype; the
    angle is position * inv_freq in the working dtype.
    qwen-infer/src/model.rs:144-163.
    """
    inv_freq = [1.0 / (float(theta) ** (i / head_dim)) for i in range(0, head_dim, 2)]
    inv_freq = torch.tensor(inv_freq, dtype=torch.float64).to(dtype).reshape(1, -1)
    positions = torch.arange(n_positions, dtype=dtype).reshape(-1, 1)
    freqs = positions @ inv_freq
    return freqs.cos(), freqs.sin()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Half-split rotation: (x1*cos - x2*sin, x2*cos + x1*sin).

    x is (heads, seq, head_dim); cos/sin are the table rows of the positions,
    (seq, head_dim/2).  qwen-infer/src/model.rs:131-137,166-172.
    """
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """kv head h serves q heads h*n_rep .. (h+1)*n_rep-1.  model.rs:571-580."""
    if n_rep == 1:
        return x
    n_kv, seq, dim = x.shape
    return x.unsqueeze(1).expand(n_kv, n_rep, seq, dim).reshape(n_kv * n_rep, seq, dim)


def mask_value(query: int, key: int, window: int | None) -> float:
    """0 or -inf.  qwen-infer/src/model.rs:119-129."""
    if key > query:
        return -math.inf
    if window is not None and key + window < query:
        return -math.inf
    return 0.0


def attention_mask(q_positions, k_positions, window: int | None, dtype=torch.float32) -> torch.Tensor:
    """Additive (q, k) mask.  qwen-infer/src/model.rs:923-940."""
    rows = [[mask_value(int(q), int(k), window) for k in k_positions] for q in q_positions]
    return torch.tensor(rows, dtype=dtype)


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """softmax(q k^T / sqrt(d) + mask) v, heads first: (heads, seq, d).

    The scale is applied after the product.  model.rs:317-323.
    """
    scale = 1.0 / math.sqrt(q.shape[-1])
    scores = (q @ k.transpose(-1, -2)) * scale
    weights = torch.softmax(scores + mask, dim=-1)
    return weights @ v


def self_attention(x, tensors, prefix, n_heads, n_kv_heads, head_dim, cos, sin, positions, window):
    """q/k/v with bias, RoPE on q and k, GQA attention, o_proj without bias.

    x is (seq, hidden); positions are the absolute positions of its rows.
    qwen-infer/src/model.rs:279-328.
    """
    seq = x.shape[0]
    q = linear(x, tensors[f"{prefix}.q_proj.weight"], tensors[f"{prefix}.q_proj.bias"])
    k = linear(x, tensors[f"{prefix}.k_proj.weight"], tensors[f"{prefix}.k_proj.bias"])
    v = linear(x, tensors[f"{prefix}.v_proj.weight"], tensors[f"{prefix}.v_proj.bias"])
    q = q.reshape(seq, n_heads, head_dim).transpose(0, 1)
    k = k.reshape(seq, n_kv_heads, head_dim).transpose(0, 1)
    v = v.reshape(seq, n_kv_heads, head_dim).transpose(0, 1)
    rows = torch.as_tensor(positions, dtype=torch.long)
    q = apply_rope(q, cos[rows], sin[rows])
    k = apply_rope(k, cos[rows], sin[rows])
    groups = n_heads // n_kv_heads
    k = repeat_kv(k, groups)
    v = repeat_kv(v, groups)
    mask = attention_mask(positions, positions, window, dtype=x.dtype)
    mixed = attend(q, k, v, mask)
    mixed = mixed.transpose(0, 1).reshape(seq, n_heads * head_dim)
    return linear(mixed, tensors[f"{prefix}.o_proj.weight"])


def silu(x: torch.Tensor) -> torch.Tensor:
    """x * sigmoid(x).  qwen-infer/src/model.rs:244."""
    return x * torch.sigmoid(x)


def mlp(x, tensors, prefix):
    """down(silu(gate(x)) * up(x)), no biases.  model.rs:245-249."""
    gated = silu(linear(x, tensors[f"{prefix}.gate_proj.weight"]))
    up = linear(x, tensors[f"{prefix}.up_proj.weight"])
    return linear(gated * up, tensors[f"{prefix}.down_proj.weight"])


def window_for_layer(cfg: dict, index: int) -> int | None:
    """model.rs:909-915."""
    if cfg.get("use_sliding_window", False) and index >= cfg["max_window_layers"]:
        return int(cfg["sliding_window"])
    return None


def decoder_layer(x, cfg, tensors, index, cos, sin, positions):
    """x + attn(norm1(x)), then + mlp(norm2(.)).  model.rs:615-622."""
    prefix = f"model.layers.{index}"
    eps = cfg["rms_norm_eps"]
    n_heads = cfg["num_attention_heads"]
    head_dim = cfg["hidden_size"] // n_heads
    residual = x
    h = rms_norm(x, tensors[f"{prefix}.input_layernorm.weight"], eps)
    h = self_attention(h, tensors, f"{prefix}.self_attn", n_heads, cfg["num_key_value_heads"],
                       head_dim, cos, sin, positions, window_for_layer(cfg, index))
    x = h + residual
    residual = x
    h = rms_norm(x, tensors[f"{prefix}.post_attention_layernorm.weight"], eps)
    h = mlp(h, tensors, f"{prefix}.mlp")
    return h + residual


def hidden_states(cfg, tensors, ids, first_position: int = 0) -> torch.Tensor:
    """Final-norm hidden states of the whole sequence, (seq, hidden).

    model.rs:832-848 (`forward_hidden`: embedding, layers, `model.norm`).
    """
    dtype = tensors["model.embed_tokens.weight"].dtype
    n_heads = cfg["num_attention_heads"]
    head_dim = cfg["hidden_size"] // n_heads
    positions = list(range(first_position, first_position + len(ids)))
    if positions[-1] >= cfg["max_position_embeddings"]:
        raise ValueError("positions exceed max_position_embeddings")  # model.rs:896-905
    cos, sin = rope_tables(cfg["rope_theta"], head_dim, cfg["max_position_embeddings"], dtype)
    x = tensors["model.embed_tokens.weight"][torch.as_tensor(ids, dtype=torch.long)]
    for index in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, cfg, tensors, index, cos, sin, positions)
    return rms_norm(x, tensors["model.norm.weight"], cfg["rms_norm_eps"])


def all_logits(cfg, tensors, ids, first_position: int = 0) -> torch.Tensor:
    """Logits at every position, (seq, vocab).

    Tied head: hidden @ embed^T; untied: lm_head.  model.rs:1210-1242 (the
    reference keeps the last row only; every row is the same product).
    """
    hidden = hidden_states(cfg, tensors, ids, first_position)
    if cfg["tie_word_embeddings"]:
        return hidden @ tensors["model.embed_tokens.weight"].t()
    return linear(hidden, tensors["lm_head.weight"])


# --------------------------------------------------------------------- sampling
def greedy_token(logits) -> int:
    """First maximum wins (`>`).  qwen-infer/src/sample.rs:43-56."""
    values = [float(v) for v in logits]
    if not values:
        raise ValueError("no logits to sample")
    best_at, best = 0, -math.inf
    for index, value in enumerate(values):
        if value > best:
            best, best_at = value, index
    return best_at


def sample_token(logits, temperature: float, top_p: float, uniform: float) -> int:
    """Temperature + nucleus draw with a given uniform number in [0,1).

    qwen-infer/src/sample.rs:68-137, float32 arithmetic.  `uniform` stands for
    `rng.random::<f32>()`.
    """
    import numpy as np

    values = np.asarray(logits, dtype=np.float32)
    if values.size == 0:
        raise ValueError("no logits to sample")
    if not math.isfinite(temperature) or temperature < 0:
        raise ValueError("bad temperature")
    if not math.isfinite(top_p) or top_p < 0:
        raise ValueError("bad top_p")
    if temperature == 0:
        return greedy_token(values)
    f32 = np.float32
    max_logit = values.max()
    weight = np.exp((values - max_logit) / f32(temperature)).astype(np.float32)
    order = sorted(range(values.size), key=lambda i: (-float(values[i]), i))
    if top_p >= 1.0:
        cutoff = len(order)
    else:
        total = f32(0)
        for w in weight:
            total = f32(total + w)
        if total == 0 or not math.isfinite(total):
            return greedy_token(values)
        cumulative, keep = f32(0), 1
        for k, index in enumerate(order):
            cumulative = f32(cumulative + f32(weight[index] / total))
            keep = k + 1
            if cumulative >= f32(top_p):
                break
        cutoff = keep
    kept = order[:cutoff]
    kept_sum = f32(0)
    for index in kept:
        kept_sum = f32(kept_sum + weight[index])
    if kept_sum == 0 or not math.isfinite(kept_sum):
        return greedy_token(values)
    threshold = f32(f32(uniform) * kept_sum)
    for index in kept:
        mass = weight[index]
        if threshold < mass:
            return index
        threshold = f32(threshold - mass)
    return kept[-1]


def greedy_generate(cfg, tensors, prompt, new_tokens: int):
    """Argmax one step and append, recomputing everything.  lib.rs:116-130."""
    ids = list(prompt)
    out = []
    for _ in range(new_tokens):
        nxt = greedy_token(all_logits(cfg, tensors, ids)[-1])
        out.append(nxt)
        ids.append(nxt)
    return out
