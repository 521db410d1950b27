"""Reader and writer of the safetensors container: 8 bytes of header length (little endian), a
JSON header {name: {dtype, shape, data_offsets}}, then the bytes. Tensors are read by name
through a memory map, so a large file is never held whole."""

from __future__ import annotations

import json
import mmap
import struct
from pathlib import Path

import numpy as np
import torch

# name in the file -> (numpy type used to view the bytes, torch type of the result)
_DTYPES = {
    "F32": (np.dtype("<f4"), torch.float32),
    "F64": (np.dtype("<f8"), torch.float64),
    "F16": (np.dtype("<f2"), torch.float16),
    "BF16": (np.dtype("<i2"), torch.bfloat16),
    "I64": (np.dtype("<i8"), torch.int64),
    "I32": (np.dtype("<i4"), torch.int32),
    "I16": (np.dtype("<i2"), torch.int16),
    "I8": (np.dtype("i1"), torch.int8),
    "U8": (np.dtype("u1"), torch.uint8),
    "BOOL": (np.dtype("u1"), torch.bool),
}
_NAMES = {t: n for n, (_, t) in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    def __init__(self, path):
        self.path = Path(path)
        if not self.path.is_file():
            raise SafetensorsError(f"{self.path} does not exist")
        size = self.path.stat().st_size
        with open(self.path, "rb") as f:
            head = f.read(8)
            if len(head) < 8:
                raise SafetensorsError(f"{self.path} is too short to be a safetensors file")
            (header_len,) = struct.unpack("<Q", head)
            if header_len > size - 8:
                raise SafetensorsError(f"{self.path}: the header length {header_len} exceeds the file")
            try:
                header = json.loads(f.read(header_len))
            except (json.JSONDecodeError, UnicodeDecodeError) as error:
                raise SafetensorsError(f"{self.path}: the header is not valid JSON ({error})") from None
            self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None
        self._data_start = 8 + header_len
        self.metadata = header.pop("__metadata__", None)
        self.entries: dict[str, dict] = {}
        problems = []
        for name, info in header.items():
            dtype, shape, offsets = info.get("dtype"), info.get("shape"), info.get("data_offsets")
            if dtype not in _DTYPES:
                problems.append(f"{name}: unknown dtype {dtype!r}")
                continue
            count = int(np.prod(shape)) if shape else 1
            begin, end = offsets
            if end - begin != count * _DTYPES[dtype][0].itemsize:
                problems.append(f"{name}: {end - begin} bytes do not hold shape {shape} of {dtype}")
            elif begin < 0 or self._data_start + end > size:
                problems.append(f"{name}: bytes [{begin}, {end}) lie outside the file (truncated?)")
            else:
                self.entries[name] = {"dtype": dtype, "shape": tuple(shape), "offsets": (begin, end)}
        if problems:
            raise SafetensorsError(f"{self.path}: " + "; ".join(problems))

    def names(self) -> list[str]:
        return list(self.entries)

    def shape(self, name: str) -> tuple:
        return self.entries[name]["shape"]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name]["dtype"]][1]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (copy it before the file is closed)."""
        info = self.entries[name]
        np_dtype, torch_dtype = _DTYPES[info["dtype"]]
        begin, end = info["offsets"]
        array = np.frombuffer(self._map, dtype=np_dtype, count=(end - begin) // np_dtype.itemsize, offset=self._data_start + begin)
        tensor = torch.from_numpy(array.reshape(info["shape"]))  # read-only view; torch warns once
        if torch_dtype in (torch.bfloat16, torch.bool):
            tensor = tensor.view(torch_dtype)
        return tensor


def write_safetensors(path, tensors: dict, metadata: dict | None = None) -> None:
    header, offset = {}, 0
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    ordered = []
    for name, tensor in tensors.items():
        tensor = tensor.detach().cpu().contiguous()
        if tensor.dtype not in _NAMES:
            raise SafetensorsError(f"{name}: cannot store {tensor.dtype}")
        nbytes = tensor.numel() * tensor.element_size()
        header[name] = {"dtype": _NAMES[tensor.dtype], "shape": list(tensor.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
        ordered.append(tensor)
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for tensor in ordered:
            if tensor.dtype == torch.bfloat16:
                tensor = tensor.view(torch.int16)
            elif tensor.dtype == torch.bool:
                tensor = tensor.view(torch.uint8)
            f.write(tensor.numpy().tobytes())
