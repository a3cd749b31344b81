"""Reader and writer for the safetensors container (8-byte header length, JSON header, raw data).

The reader maps the file and hands out tensors by name without touching the
rest; the writer lays tensors out in name order.  Only the dtypes a model file
holds are known: BF16, F16, F32, F64, I64, I32, I16, I8, U8, BOOL.
"""
from __future__ import annotations

import json
import mmap
import os
import struct

import torch

_DTYPES = {
    "BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """A mapped safetensors file: `names()`, `info(name)` and `tensor(name)`."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except FileNotFoundError:
            raise SafetensorsError(f"no weight file at {path}") from None
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path} is truncated: {size} bytes, no header length")
        (header_len,) = struct.unpack("<Q", self._fh.read(8))
        if 8 + header_len > size:
            raise SafetensorsError(f"{path} is truncated: header of {header_len} bytes does not fit in {size}")
        try:
            header = json.loads(self._fh.read(header_len))
        except (UnicodeDecodeError, json.JSONDecodeError) as err:
            raise SafetensorsError(f"{path} has an unreadable header: {err}") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._entries = header
        self._data_start = 8 + header_len
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_COPY)
        data_len = size - self._data_start
        for name, entry in header.items():
            begin, end = entry["data_offsets"]
            if entry["dtype"] not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name} has unsupported dtype {entry['dtype']}")
            if not (0 <= begin <= end <= data_len):
                raise SafetensorsError(f"{path} is truncated: tensor {name} ends at byte {end} of {data_len}")
            count = 1
            for dim in entry["shape"]:
                count *= dim
            if count * _DTYPES[entry["dtype"]].itemsize != end - begin:
                raise SafetensorsError(f"{path}: tensor {name} of shape {entry['shape']} does not fill its "
                                       f"{end - begin} bytes")

    def names(self) -> list[str]:
        return list(self._entries)

    def info(self, name: str) -> tuple[tuple[int, ...], torch.dtype]:
        entry = self._entries[name]
        return tuple(entry["shape"]), _DTYPES[entry["dtype"]]

    def tensor(self, name: str) -> torch.Tensor:
        """A tensor that views the mapping (copy-on-write); clone or move it to keep it."""
        entry = self._entries[name]
        shape, dtype = tuple(entry["shape"]), _DTYPES[entry["dtype"]]
        begin, end = entry["data_offsets"]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        count = (end - begin) // dtype.itemsize
        flat = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self._data_start + begin)
        return flat.reshape(shape)

    def close(self) -> None:
        # Tensors handed out may still view the mapping; let the garbage collector end it.
        self._fh.close()


def save_safetensors(path: str, tensors: dict[str, torch.Tensor], metadata: dict[str, str] | None = None) -> None:
    header: dict = {}
    if metadata:
        header["__metadata__"] = metadata
    offset = 0
    order = sorted(tensors)
    for name in order:
        tensor = tensors[name]
        if tensor.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store {name} of dtype {tensor.dtype}")
        nbytes = tensor.numel() * tensor.dtype.itemsize
        header[name] = {"dtype": _NAMES[tensor.dtype], "shape": list(tensor.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(blob)))
        fh.write(blob)
        for name in order:
            tensor = tensors[name].detach().cpu().contiguous()
            fh.write(tensor.reshape(-1).view(torch.uint8).numpy().tobytes())
