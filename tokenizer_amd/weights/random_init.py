"""Random-weights mode: a model folder from a configuration and a seed.

Every tensor is drawn from its own generator keyed by (seed, tensor name), so
the values of a tensor do not depend on which other tensors exist.  Matrices,
biases and the embedding are N(0, std) rounded to bfloat16 (the dtype model
files are stored in); norm scales are 1, or 1 + spread * N(0, 1) when a spread
is asked for (tests do: with every scale equal to 1 two norms could be swapped,
or one left out, and no logit would change).
"""
from __future__ import annotations

import hashlib
import os

import torch

from ..config.base import ModelConfig
from ..parts.spec import TensorSpec
from .safetensors_io import save_safetensors


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return gen


def random_tensor(name: str, spec: TensorSpec, seed: int, norm_spread: float = 0.0) -> torch.Tensor:
    if spec.role == "table":
        return torch.zeros(spec.shape, dtype=torch.int32)
    if spec.init == "ones":
        if not norm_spread:
            return torch.ones(spec.shape, dtype=torch.bfloat16)
        noise = torch.empty(spec.shape, dtype=torch.float32).normal_(0.0, 1.0, generator=_generator(seed, name))
        return (1.0 + float(norm_spread) * noise).to(torch.bfloat16)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=torch.bfloat16)
    if spec.init != "normal":
        raise ValueError(f"unknown init {spec.init!r} for {name}")
    values = torch.empty(spec.shape, dtype=torch.float32)
    values.normal_(0.0, spec.std, generator=_generator(seed, name))
    # A tensor that is kept as stored is written in 32-bit: that is what such tensors (router weights,
    # decay rates and the like) are stored in, and the loader then leaves it so in both modes.
    return values if spec.role == "keep" else values.to(torch.bfloat16)


def random_tensors(expected: dict[str, TensorSpec], seed: int, norm_spread: float = 0.0) -> dict[str, torch.Tensor]:
    return {name: random_tensor(name, spec, seed, norm_spread) for name, spec in expected.items()}


def write_random_model(config: ModelConfig, seed: int, folder: str, norm_spread: float = 0.0) -> str:
    """Write config.json and model.safetensors for `config` with weights from `seed`.  `norm_spread`: how far
    the norms' scales lie from 1 (standard deviation; 0 = all equal to 1)."""
    from ..config.registry import get_architecture
    from ..parts.model import expected_tensors

    spec = get_architecture(config.architecture).build_spec(config)
    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    save_safetensors(os.path.join(folder, "model.safetensors"),
                     random_tensors(expected_tensors(spec), seed, norm_spread),
                     metadata={"format": "pt", "seed": str(seed)})
    return folder
