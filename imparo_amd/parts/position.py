"""Position encodings. A position part owns a table of inverse frequencies
and says which dimensions make a pair (`interleaved` False: i with i +
rotary_dim/2; True: 2i with 2i + 1); the attention mixer hands both to the
fused norm+rotation kernel together with each token's absolute position.

NeoX rotation: dimension i pairs with i + rotary_dim/2, inv_i =
base^(-2i/rotary_dim), angle = position * inv_i
(/root/reference/crates/imparo-cpu/src/ops.rs:551-569)."""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from ..config.plan import PartSpec
from .registry import register_part


class RopeNeox:
    role = "position"
    interleaved = False

    def __init__(self, spec: PartSpec, device: torch.device):
        self.rotary_dim = int(spec["rotary_dim"])
        self.base = float(spec["base"])
        if self.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {self.rotary_dim}")
        half = self.rotary_dim // 2
        i = np.arange(half, dtype=np.float32)
        expo = (np.float32(-2.0) * i / np.float32(self.rotary_dim)).astype(np.float32)
        inv = np.power(np.float32(self.base), expo).astype(np.float32)
        factors = spec.get("frequency_factors")
        if factors is not None:      # divides theta per pair
            inv = (inv / np.asarray(factors, dtype=np.float32)).astype(np.float32)
        self.inv_freq: Optional[torch.Tensor] = torch.from_numpy(inv).to(device)


class NoPosition:
    """No rotation: keys are cached as the norm leaves them."""
    role = "position"

    interleaved = False

    def __init__(self, spec: PartSpec, device: torch.device):
        self.rotary_dim = 0
        self.inv_freq = None


register_part("position", "rope_neox", RopeNeox)
register_part("position", "none", NoPosition)
