"""Reading and writing the safetensors container.

The format: 8 bytes little-endian header length, a JSON header mapping tensor
name -> {dtype, shape, data_offsets}, then the raw little-endian tensor bytes.
Reading memory-maps the file, so a tensor costs host memory only when touched.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, List, Tuple

import torch

_DTYPES = {
    "F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16,
    "I32": torch.int32, "I64": torch.int64, "F64": torch.float64,
    "U8": torch.uint8, "I8": torch.int8, "I16": torch.int16, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """A memory-mapped safetensors file: `entries` lists what it holds,
    `tensor(name)` returns a CPU tensor viewing the mapped bytes."""

    def __init__(self, path: str):
        self.path = path
        self._file = open(path, "rb")
        head = self._file.read(8)
        if len(head) != 8:
            raise SafetensorsError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", head)
        size = self._file.seek(0, 2)
        if n > size - 8:
            raise SafetensorsError(f"{path}: header length {n} exceeds the file")
        self._file.seek(8)
        try:
            header = json.loads(self._file.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from None
        header.pop("__metadata__", None)
        self._base = 8 + n
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            if info["dtype"] not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {info['dtype']}")
            begin, end = info["data_offsets"]
            dtype = _DTYPES[info["dtype"]]
            shape = tuple(int(s) for s in info["shape"])
            count = 1
            for s in shape:
                count *= s
            if (not 0 <= begin <= end or end - begin != count * torch.empty((), dtype=dtype).element_size()
                    or self._base + end > size):
                raise SafetensorsError(f"{path}: tensor {name!r} has inconsistent offsets")
            self.entries[name] = (dtype, shape, begin, end)
        spans = sorted((b, e, name) for name, (_, _, b, e) in self.entries.items() if e > b)
        for (b0, e0, n0), (b1, e1, n1) in zip(spans, spans[1:]):
            if b1 < e0:
                raise SafetensorsError(f"{path}: tensors {n0!r} and {n1!r} overlap in the file")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> List[str]:
        return list(self.entries)

    def dtype(self, name: str) -> torch.dtype:
        return self.entries[name][0]

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def tensor(self, name: str) -> torch.Tensor:
        dtype, shape, begin, end = self.entries[name]
        if end == begin:
            return torch.empty(shape, dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the mapping is read-only; nothing writes through it
            flat = torch.frombuffer(self._map, dtype=dtype, count=(end - begin) // _elem(dtype),
                                    offset=self._base + begin)
        return flat.reshape(shape)

    def close(self) -> None:
        self._map = None
        self._file.close()


def _elem(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


def save_file(tensors: Dict[str, torch.Tensor], path: str) -> None:
    """Writes CPU tensors to `path`, names sorted, data 8-byte aligned."""
    header = {}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r} has dtype {t.dtype}, which safetensors cannot hold")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    # written beside the target and renamed over it: a file that is mapped
    # somewhere (even as the source of these tensors) is never truncated
    tmp = f"{path}.tmp{os.getpid()}"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            f.write(t.view(torch.uint8).reshape(-1).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
