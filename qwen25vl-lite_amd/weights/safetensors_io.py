"""Reading and writing the safetensors container, by tensor name.

The format is an 8-byte little-endian header length, a JSON header
``{name: {"dtype", "shape", "data_offsets": [begin, end]}}`` and the raw little-endian data.
The reader maps the file into memory and hands out one tensor at a time, so a checkpoint is
never held twice in host memory (the reference streams its shards the same way, reference
src/qwen25vl_lite/model.py:312-348).
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterator, List, Tuple

import torch

__all__ = ["SafetensorsFile", "write_safetensors", "checkpoint_shards"]

_DTYPES = {
    "F32": torch.float32,
    "BF16": torch.bfloat16,
    "F16": torch.float16,
    "F64": torch.float64,
    "I64": torch.int64,
    "I32": torch.int32,
    "I16": torch.int16,
    "I8": torch.int8,
    "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    """One safetensors file, memory-mapped; tensors are read by name."""

    def __init__(self, path: str):
        self.path = path
        self._fh = open(path, "rb")
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise ValueError(f"{path}: too short to be a safetensors file")
        (header_len,) = struct.unpack("<Q", self._fh.read(8))
        if header_len <= 0 or 8 + header_len > size:
            raise ValueError(f"{path}: header length {header_len} does not fit the file")
        header = json.loads(self._fh.read(header_len).decode("utf-8"))
        header.pop("__metadata__", None)
        self._base = 8 + header_len
        self._entries: Dict[str, dict] = header
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_COPY) if size else None
        for name, entry in header.items():
            if entry["dtype"] not in _DTYPES:
                raise ValueError(f"{path}: tensor {name!r} has the unknown dtype {entry['dtype']!r}")
            begin, end = entry["data_offsets"]
            if not (0 <= begin <= end and self._base + end <= size):
                raise ValueError(f"{path}: tensor {name!r} lies outside the file")

    def keys(self) -> List[str]:
        return list(self._entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(int(d) for d in self._entries[name]["shape"])

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self._entries[name]["dtype"]]

    def tensor(self, name: str) -> torch.Tensor:
        """A host tensor that views the mapped file (copy it before the file is closed)."""
        entry = self._entries[name]
        begin, end = entry["data_offsets"]
        dtype = _DTYPES[entry["dtype"]]
        shape = tuple(int(d) for d in entry["shape"])
        count = 1
        for d in shape:
            count *= d
        if count * torch.empty((), dtype=dtype).element_size() != end - begin:
            raise ValueError(f"{self.path}: tensor {name!r} has {end - begin} bytes for shape {shape}")
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        view = memoryview(self._map)[self._base + begin:self._base + end]
        return torch.frombuffer(view, dtype=dtype, count=count).reshape(shape)

    def items(self) -> Iterator[Tuple[str, torch.Tensor]]:
        for name in self._entries:
            yield name, self.tensor(name)

    def close(self) -> None:
        # Tensors handed out may still view the map; dropping our references is enough,
        # the map goes when the last view does.
        self._map = None
        self._fh.close()

    def __enter__(self) -> "SafetensorsFile":
        return self

    def __exit__(self, *exc) -> None:
        self.close()


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor]) -> None:
    """Write tensors (host or device) under their names, in the given order."""
    header: Dict[str, dict] = {}
    offset = 0
    order = list(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise ValueError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as fh:
        fh.write(struct.pack("<Q", len(blob)))
        fh.write(blob)
        for name in order:
            t = tensors[name].detach().to("cpu").contiguous()
            if t.numel():
                fh.write(t.view(torch.uint8).reshape(-1).numpy().tobytes()
                         if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)


def checkpoint_shards(model_dir: str) -> List[str]:
    """The safetensors files of a model folder: those the index names, else
    ``model.safetensors`` (reference model.py:314-327)."""
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as fh:
            weight_map = json.load(fh)["weight_map"]
        return [os.path.join(model_dir, s) for s in sorted(set(weight_map.values()))]
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    raise FileNotFoundError(
        f"no safetensors weights under {model_dir!r}: expected model.safetensors or model.safetensors.index.json")
