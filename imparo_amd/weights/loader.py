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

import json
import os
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile

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


INDEX_FILE = "model.safetensors.index.json"


class _Files:
    """The open files of a checkpoint: one model.safetensors, or the shards an
    index names. Kept alive while views of their mappings are in use."""

    def __init__(self, files):
        self.files = files

    def close(self) -> None:
        for f in self.files:
            f.close()


def _open_checkpoint(model_dir: str):
    """-> (label for messages, {tensor name: file that holds it}, _Files).
    A folder holds either `model.safetensors` or `model.safetensors.index.json`,
    whose `weight_map` sends every tensor name to a shard file beside it."""
    single = os.path.join(model_dir, WEIGHTS_FILE)
    index = os.path.join(model_dir, INDEX_FILE)
    if os.path.isfile(single):
        f = SafetensorsFile(single)
        return single, {name: f for name in f.names()}, _Files([f])
    if not os.path.isfile(index):
        raise FileNotFoundError(f"{model_dir} holds neither {WEIGHTS_FILE} nor {INDEX_FILE}")
    with open(index, "r", encoding="utf-8") as fh:
        weight_map = json.load(fh).get("weight_map")
    if not isinstance(weight_map, dict) or not weight_map:
        raise SafetensorsError(f"{index}: no weight_map of tensor name -> shard file")
    shards: Dict[str, SafetensorsFile] = {}
    where: Dict[str, SafetensorsFile] = {}
    try:
        for name, shard in sorted(weight_map.items()):
            if not isinstance(shard, str) or os.path.basename(shard) != shard:
                raise SafetensorsError(f"{index}: {name} is mapped to {shard!r}, which is no file beside the index")
            if shard not in shards:
                path = os.path.join(model_dir, shard)
                if not os.path.isfile(path):
                    raise FileNotFoundError(f"{index} names the shard {shard}, which does not exist")
                shards[shard] = SafetensorsFile(path)
            if name not in shards[shard].entries:
                raise SafetensorsError(f"{index}: {name} is mapped to {shard}, which does not hold it")
            where[name] = shards[shard]
        # a tensor that a shard holds but the index does not name is in the checkpoint all the same
        for shard, f in shards.items():
            for name in f.names():
                where.setdefault(name, f)
    except Exception:
        for f in shards.values():
            f.close()
        raise
    return index, where, _Files(list(shards.values()))


def load_weights(model_dir: str, declared: Dict[str, TensorDecl],
                 same_as: Optional[Dict[str, str]] = None) -> Dict[str, torch.Tensor]:
    """Reads the checkpoint in `model_dir` (`model.safetensors`, or the shards
    of `model.safetensors.index.json`) against `declared`; returns CPU tensors
    by name, or raises one WeightsError listing every fault. `same_as` maps a
    name nobody declared to a declared one it may restate (a stored head beside
    a tied embedding): such a tensor is accepted if it equals the other
    bit for bit, and is an unexpected tensor otherwise."""
    path, where, files = _open_checkpoint(model_dir)
    have = set(where)
    want = set(declared)
    missing = want - have
    unexpected = have - want
    for name in sorted(unexpected):
        twin = (same_as or {}).get(name)
        if twin in where and twin in want:
            a, b = where[name], where[twin]
            if (a.dtype(name), a.shape(name)) == (b.dtype(twin), b.shape(twin)) and \
                    torch.equal(a.tensor(name).view(torch.uint8), b.tensor(twin).view(torch.uint8)):
                unexpected.discard(name)
    wrong_shape, wrong_dtype = [], []
    for name in want & have:
        decl = declared[name]
        f = where[name]
        if tuple(f.shape(name)) != tuple(decl.shape):
            wrong_shape.append((name, tuple(decl.shape), tuple(f.shape(name))))
        dt = f.dtype(name)
        ok = dt in _INTS if decl.role == "table" else dt in _FLOATS
        if not ok:
            wrong_dtype.append((name, str(dt)))
    if missing or unexpected or wrong_shape or wrong_dtype:
        files.close()
        raise WeightsError(path, missing, unexpected, wrong_shape, wrong_dtype)
    out: Dict[str, torch.Tensor] = {}
    for name in sorted(want):
        t = where[name].tensor(name)
        if t.dtype == torch.float16:
            t = t.to(torch.bfloat16)
        elif t.dtype in _INTS and t.dtype != torch.int32:
            t = t.to(torch.int32)
        out[name] = t
    out["__file__"] = files   # keeps the mappings alive while views of them are in use
    return out
