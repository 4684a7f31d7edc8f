"""Reading and writing the safetensors format without any other package.

Layout of a file: 8 bytes little-endian header length N, N bytes of JSON
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`,
then the raw little-endian tensor bytes, offsets relative to the end of the
header.  The reference never reads a file: it borrows the tensors of a loaded
transformers model by the same names (engine/model.py:190-229).
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, Mapping, Tuple

import torch

_TORCH_OF = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAME_OF = {v: k for k, v in _TORCH_OF.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """A memory-mapped safetensors file: `entries` without touching the data,
    `tensor(name)` as a CPU tensor that views the mapping."""

    def __init__(self, path: str) -> None:
        self.path = path
        self._handle = open(path, "rb")
        size = os.fstat(self._handle.fileno()).st_size
        if size < 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (header_len,) = struct.unpack("<Q", self._handle.read(8))
        if header_len > size - 8:
            raise SafetensorsError(f"{path}: header length {header_len} exceeds the file")
        try:
            header = json.loads(self._handle.read(header_len).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as err:
            raise SafetensorsError(f"{path}: header is not JSON ({err})") from err
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + header_len
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            begin, end = info["data_offsets"]
            if info["dtype"] not in _TORCH_OF:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {info['dtype']}")
            if end > size - self._data_start or begin > end:
                raise SafetensorsError(f"{path}: tensor '{name}' lies outside the file")
            self.entries[name] = (info["dtype"], tuple(int(d) for d in info["shape"]), begin, end)
        self._map = mmap.mmap(self._handle.fileno(), 0, access=mmap.ACCESS_COPY) if size else None

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return _TORCH_OF[self.entries[name][0]]

    def tensor(self, name: str) -> torch.Tensor:
        code, shape, begin, end = self.entries[name]
        dtype = _TORCH_OF[code]
        count = 1
        for d in shape:
            count *= d
        if count == 0:
            return torch.empty(shape, dtype=dtype)
        want = count * torch.empty((), dtype=dtype).element_size()
        if end - begin != want:
            raise SafetensorsError(
                f"{self.path}: tensor '{name}' holds {end - begin} bytes, its shape needs {want}")
        flat = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self._data_start + begin)
        return flat.view(shape)

    def close(self) -> None:
        self._handle.close()


def save_file(tensors: Mapping[str, torch.Tensor], path: str, metadata: Mapping[str, str] | None = None) -> None:
    """Write `tensors` (CPU or device tensors) as one safetensors file."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAME_OF:
            raise SafetensorsError(f"tensor '{name}' has a dtype safetensors cannot hold: {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAME_OF[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(blob)))
        handle.write(blob)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            if t.numel():
                handle.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else
                             t.reshape(1).view(torch.uint8).numpy().tobytes())
