"""Random-weights mode: a configuration and a seed -> a model folder.

Every tensor is drawn from its own generator, seeded by (seed, tensor name),
so the folder does not depend on the order tensors are declared in. The
distributions: matrices and embeddings N(0, 0.02); depthwise conv taps
N(0, 0.1); norm weights 1 + U(-0.1, 0.1); biases N(0, 0.02).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Iterable

import torch

from ..config import plan_from_config
from .loader import TensorDecl, WEIGHTS_FILE
from .safetensors_io import save_file


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFF_FFFF_FFFF_FFFF)
    return g


def random_tensor(seed: int, name: str, decl: TensorDecl, init: str) -> torch.Tensor:
    g = _generator(seed, name)
    if init == "norm":
        return 1.0 + (torch.rand(decl.shape, generator=g) * 0.2 - 0.1)
    std = 0.1 if init == "conv" else 0.02
    return torch.randn(decl.shape, generator=g) * std


def write_random_model(config: Dict[str, Any], seed: int, out_dir: str,
                       dtype: torch.dtype = torch.bfloat16,
                       keep_float32: Iterable[str] = (), layer_gain: float = 1.0) -> str:
    """Writes config.json and model.safetensors for `config` under `out_dir`.

    Tensors are generated in float32 and stored as `dtype`; a tensor whose name
    contains one of `keep_float32` is stored in float32. With the stated
    spreads a small model's layers add little to the embedding, and with a tied
    head its greedy continuation is one token repeated; `layer_gain` draws the
    matrices of the layers (not the embedding, not the head) that many times
    wider, so that the continuation depends on everything the layers compute.
    """
    from ..engine.model import declared_tensors   # parts say what they read
    _, plan = plan_from_config(config)
    declared = declared_tensors(plan)
    keep = tuple(keep_float32)
    from ..parts import part_class
    outer = set(part_class("embedding", plan.embedding.kind).declare(plan.embedding))
    outer |= set(part_class("head", plan.head.kind).declare(plan.head))
    tensors = {}
    for name, (decl, init) in declared.items():
        t = random_tensor(seed, name, decl, init)
        if layer_gain != 1.0 and init == "matrix" and name not in outer:
            t = t * layer_gain
        tensors[name] = t if any(k in name for k in keep) else t.to(dtype)
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config, f, indent=1, sort_keys=True)
    save_file(tensors, os.path.join(out_dir, WEIGHTS_FILE))
    return out_dir
