"""Weights by tensor name, checked against what the model's parts expect.

The file is matched to the expectation in one pass and every problem is
reported together: missing tensors, unexpected tensors and wrong shapes.
Tensors the model does not read are no reason to refuse a file that holds
everything else (the reference's loader takes what it asks for by name and never
looks at the rest, qwen-infer/src/model.rs:776-786: a tied model saved with a
redundant `lm_head.weight`, an export with `rotary_emb.inv_freq` buffers): alone
they are a warning; beside a real misfit they are listed in the same error,
since a misnamed tensor shows up as one missing and one unexpected name.
`strict=True` makes them an error on their own.
Tensors are not renamed; a part that wants two matrices side by side joins
them itself after loading (the reference keeps q, k, v and gate, up apart,
qwen-infer/src/model.rs:263-276).
"""
from __future__ import annotations

import json
import os
import warnings

import torch

from ..parts.spec import TensorSpec
from .safetensors_io import SafetensorsError, SafetensorsFile


class UnexpectedTensors(UserWarning):
    """The weight file holds tensors that the model does not read."""


class WeightError(ValueError):
    """The weight file does not hold what the model needs."""

    def __init__(self, path, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=(), other=()):
        self.path = path
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)   # (name, found, wanted)
        self.wrong_dtype = list(wrong_dtype)   # (name, found)
        self.other = list(other)
        lines = [f"weights in {path} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(f)}, wanted {list(w)}" for n, f, w in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  unusable dtype ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n} is {d}" for n, d in self.wrong_dtype))
        lines.extend(f"  {msg}" for msg in self.other)
        super().__init__("\n".join(lines))


_FLOATS = (torch.bfloat16, torch.float16, torch.float32, torch.float64)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


def stored_form(tensor: torch.Tensor, spec: TensorSpec, compute_dtype: torch.dtype) -> torch.Tensor:
    """How a loaded tensor is kept: see `TensorSpec.role`.

    Matrices feed the matrix products and are held in the compute dtype
    (bfloat16 files stay bfloat16 in bfloat16 mode and are widened, exactly, in
    float32 mode).  Vectors are widened to float32.  Integer tables become
    int32.  "keep" leaves a tensor as stored, so one stored in 32-bit stays so.
    """
    if spec.role == "matrix":
        return tensor.to(compute_dtype)
    if spec.role == "vector":
        return tensor.to(torch.float32)
    if spec.role == "table":
        return tensor.to(torch.int32)
    return tensor


def weight_path(folder: str) -> str:
    return os.path.join(folder, "model.safetensors") if os.path.isdir(folder) else folder


class ShardedWeights:
    """A model stored in several safetensors files beside `model.safetensors.index.json`, whose `weight_map`
    says which file holds which tensor (larger checkpoints are published that way; the reference reads a single
    file, qwen-infer/src/lib.rs:56-60).  Same face as `SafetensorsFile`; a shard is mapped when first asked for."""

    def __init__(self, index_path: str):
        self.path = index_path
        try:
            with open(index_path, encoding="utf-8") as fh:
                weight_map = json.load(fh)["weight_map"]
        except (OSError, ValueError, KeyError, TypeError) as err:
            raise SafetensorsError(f"{index_path} is no shard index: {err}") from None
        if not isinstance(weight_map, dict):
            raise SafetensorsError(f"{index_path}: weight_map is not an object")
        self._folder = os.path.dirname(index_path)
        self._file_of = weight_map
        self._shards: dict[str, SafetensorsFile] = {}

    def _shard(self, name: str) -> SafetensorsFile:
        file_name = self._file_of[name]
        if file_name not in self._shards:
            self._shards[file_name] = SafetensorsFile(os.path.join(self._folder, file_name))
        return self._shards[file_name]

    def names(self) -> list[str]:
        # What the shards really hold: a name the index promises but its file lacks is then reported as missing.
        return [name for name in self._file_of if name in self._shard(name)._entries]

    def info(self, name: str):
        return self._shard(name).info(name)

    def tensor(self, name: str):
        return self._shard(name).tensor(name)

    def close(self) -> None:
        for shard in self._shards.values():
            shard.close()


def open_weights(folder: str):
    """The weights of a model folder: `model.safetensors`, or the shards that `model.safetensors.index.json` lists."""
    path = weight_path(folder)
    index = path + ".index.json"
    if not os.path.exists(path) and os.path.exists(index):
        return ShardedWeights(index)
    return SafetensorsFile(path)


def load_weights(folder: str, expected: dict[str, TensorSpec], compute_dtype: torch.dtype,
                 device: torch.device | str = "cpu", strict: bool = False) -> dict[str, torch.Tensor]:
    """Load the tensors in `expected`, or raise one `WeightError` naming every misfit (missing, wrong shape,
    unusable dtype, and the unexpected names beside them).  Unexpected tensors alone: an `UnexpectedTensors`
    warning that lists them, or the same error with `strict=True`."""
    path = weight_path(folder)
    try:
        source = open_weights(folder)
        path = source.path
        names = set(source.names())
    except SafetensorsError as err:
        raise WeightError(path, other=[str(err)]) from None
    missing = sorted(set(expected) - names)
    unexpected = sorted(names - set(expected))
    wrong_shape, wrong_dtype = [], []
    for name in sorted(names & set(expected)):
        shape, dtype = source.info(name)
        spec = expected[name]
        if tuple(shape) != tuple(spec.shape):
            wrong_shape.append((name, shape, spec.shape))
        if spec.role in ("matrix", "vector") and dtype not in _FLOATS:
            wrong_dtype.append((name, dtype))
        if spec.role == "table" and dtype not in _INTS:
            wrong_dtype.append((name, dtype))
    if missing or wrong_shape or wrong_dtype or (unexpected and strict):
        source.close()
        raise WeightError(path, missing, unexpected, wrong_shape, wrong_dtype)
    if unexpected:
        warnings.warn(UnexpectedTensors(f"{path} holds {len(unexpected)} tensors the model does not read: "
                                        + ", ".join(unexpected)), stacklevel=2)
    out = {}
    for name, spec in expected.items():
        out[name] = stored_form(source.tensor(name), spec, compute_dtype).to(device).contiguous()
    source.close()
    return out
