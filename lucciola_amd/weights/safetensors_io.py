"""Reading and writing the safetensors container.

Layout, as the reference parses it (src/safetensors.cc:51-87): an unsigned 64-bit
little-endian header length, a JSON header ``{name: {dtype, shape, data_offsets: [b, e]}}``
(the ``__metadata__`` entry is skipped) and the tensors' bytes from ``8 + header length`` on.
The file is memory-mapped; a tensor's bytes are touched only when it is asked for.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
import warnings
from dataclasses import dataclass
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch


class SafetensorsError(ValueError):
    pass


_DTYPE_FROM_TAG = {
    "F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64,
    "I32": torch.int32, "I64": torch.int64, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_TAG_FROM_DTYPE = {v: k for k, v in _DTYPE_FROM_TAG.items()}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: Tuple[int, ...]
    begin: int
    end: int


class SafetensorsFile:
    """A memory-mapped safetensors file; ``entries`` lists what it holds."""

    def __init__(self, path: str):
        self.path = path
        if not os.path.isfile(path):
            raise SafetensorsError(f"no such weights file: '{path}'")
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors header ({size} bytes)")
        self._fh = open(path, "rb")
        (header_len,) = struct.unpack("<Q", self._fh.read(8))
        if header_len <= 0 or 8 + header_len > size:
            self._fh.close()
            raise SafetensorsError(f"{path}: header length {header_len} does not fit the file "
                                   f"({size} bytes): truncated or not a safetensors file")
        raw = self._fh.read(header_len)
        try:
            header = json.loads(raw.decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as exc:
            self._fh.close()
            raise SafetensorsError(f"{path}: header is not valid JSON ({exc})") from exc
        self._base = 8 + header_len
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        self.entries: Dict[str, TensorEntry] = {}
        data_size = size - self._base
        for name, info in header.items():
            if name == "__metadata__":
                continue
            tag = info.get("dtype")
            if tag not in _DTYPE_FROM_TAG:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype '{tag}'")
            shape = tuple(int(s) for s in info.get("shape", ()))
            begin, end = (int(x) for x in info["data_offsets"])
            dtype = _DTYPE_FROM_TAG[tag]
            want = int(np.prod(shape, dtype=np.int64)) * torch.empty((), dtype=dtype).element_size()
            if begin < 0 or end > data_size or end - begin != want:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' {tag}{list(shape)} needs {want} bytes but its "
                    f"offsets [{begin}, {end}) give {end - begin} (data section: {data_size} bytes)")
            self.entries[name] = TensorEntry(name, dtype, shape, begin, end)

    def names(self) -> List[str]:
        return list(self.entries)

    def get(self, name: str) -> torch.Tensor:
        """The tensor as a CPU tensor that views the mapping (copy it before the file closes)."""
        entry = self.entries[name]
        count = int(np.prod(entry.shape, dtype=np.int64))
        if count == 0:
            return torch.empty(entry.shape, dtype=entry.dtype)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)   # the mapping is read-only, and is only read
            flat = torch.frombuffer(self._map, dtype=entry.dtype, count=count,
                                    offset=self._base + entry.begin)
        return flat.view(entry.shape)

    def close(self) -> None:
        try:
            self._map.close()
        except (BufferError, ValueError):
            pass  # views of the mapping are still alive; the mapping goes with them
        self._fh.close()

    def __enter__(self) -> "SafetensorsFile":
        return self

    def __exit__(self, *exc) -> None:
        self.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]]) -> None:
    """Write ``(name, tensor)`` pairs; tensors are taken one at a time and may live on any device."""
    items: List[Tuple[str, torch.Tensor]] = []
    header: Dict[str, dict] = {}
    offset = 0
    for name, tensor in tensors:
        t = tensor.detach().contiguous().cpu()
        if t.dtype not in _TAG_FROM_DTYPE:
            raise SafetensorsError(f"tensor '{name}': dtype {t.dtype} cannot be written")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TAG_FROM_DTYPE[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        items.append((name, t))
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as fh:
        fh.write(struct.pack("<Q", len(blob)))
        fh.write(blob)
        for _, t in items:
            if t.numel():
                fh.write(memoryview(t.reshape(-1).view(torch.uint8).numpy()))
    os.replace(tmp, path)
