"""Weights by tensor name.

Every part of a model declares the tensors it reads (name, shape, role); the
loader checks the file against the union of those declarations and reports
everything that is wrong in ONE error: missing names, names nobody asked for,
wrong shapes, unreadable dtypes. The reference resolves tensors the same way,
by name and with by-name errors, and reads only the arm a layer's kind needs
(/root/reference/crates/imparo-model/src/cpu_support.rs:97-175,
/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:84-122).

Floating tensors stored in 16 bits are kept in bfloat16, a tensor stored in
32 bits stays in 32 bits, integer tables become int32.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, Tuple

import torch

from .safetensors_io import SafetensorsFile

WEIGHTS_FILE = "model.safetensors"


@dataclass(frozen=True)
class TensorDecl:
    shape: Tuple[int, ...]
    role: str = "matrix"      # "matrix" | "vector" | "table" (integer)


class WeightsError(ValueError):
    """What is wrong with a weights file, all of it at once."""

    def __init__(self, path, missing, unexpected, wrong_shape, wrong_dtype):
        self.path = path
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        self.wrong_dtype = sorted(wrong_dtype)
        lines = [f"{path} does not hold the tensors this model needs:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, expected {list(want)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  unsupported dtype: {name} is {got}")
        super().__init__("\n".join(lines))


_FLOATS = (torch.float32, torch.bfloat16, torch.float16)
_INTS = (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8)


def load_weights(model_dir: str, declared: Dict[str, TensorDecl]) -> Dict[str, torch.Tensor]:
    """Reads `model_dir/model.safetensors` against `declared`; returns CPU
    tensors by name, or raises one WeightsError listing every fault."""
    path = os.path.join(model_dir, WEIGHTS_FILE)
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{path} does not exist")
    f = SafetensorsFile(path)
    have = set(f.names())
    want = set(declared)
    missing = want - have
    unexpected = have - want
    wrong_shape, wrong_dtype = [], []
    for name in want & have:
        decl = declared[name]
        if tuple(f.shape(name)) != tuple(decl.shape):
            wrong_shape.append((name, tuple(decl.shape), tuple(f.shape(name))))
        dt = f.dtype(name)
        ok = dt in _INTS if decl.role == "table" else dt in _FLOATS
        if not ok:
            wrong_dtype.append((name, str(dt)))
    if missing or unexpected or wrong_shape or wrong_dtype:
        f.close()
        raise WeightsError(path, missing, unexpected, wrong_shape, wrong_dtype)
    out: Dict[str, torch.Tensor] = {}
    for name in sorted(want):
        t = f.tensor(name)
        if t.dtype == torch.float16:
            t = t.to(torch.bfloat16)
        elif t.dtype in _INTS and t.dtype != torch.int32:
            t = t.to(torch.int32)
        out[name] = t
    out["__file__"] = f   # keeps the mapping alive while views of it are in use
    return out
