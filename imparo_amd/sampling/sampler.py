"""Picking tokens from logits.

Greedy: the smallest index attaining the maximum, NaN never wins -- the rule
the reference's host and device argmax share
(/root/reference/crates/imparo-cpu/src/ops.rs:628-640). The reference's
`sample` ignores the temperature it parses
(/root/reference/crates/imparo-server/src/main.rs:3382-3390); here a positive
temperature draws from softmax(logits / T) by inverse CDF with a uniform
number that depends only on (seed, index of the generated token), so a
request's draws do not depend on what it was batched with.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple


_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform_for(seed: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits, a pure function of (seed, index)."""
    h = _splitmix64(_splitmix64(seed & _MASK) ^ ((index * 0xD1342543DE82EF95) & _MASK))
    return (h >> 40) / float(1 << 24)


@dataclass
class SamplingParams:
    """`max_tokens` and `temperature` carry the reference's request fields of
    those names (/root/reference/crates/imparo-server/src/main.rs:1849-1872);
    temperature 0 is greedy."""
    temperature: float = 0.0
    max_tokens: int = 16
    seed: int = 0
    stop_token_ids: Tuple[int, ...] = ()


class PendingPick:
    """Token ids that the sampling kernel has been asked for. `on_device` is
    the int32 vector they land in (to feed the next step from, without
    waiting); `tokens()` waits for the copy to the host and returns them."""

    def __init__(self, on_device, host, event):
        self.on_device = on_device
        self._host = host
        self._event = event
        self._tokens: Optional[List[int]] = None

    def tokens(self) -> List[int]:
        if self._tokens is None:
            self._event.synchronize()
            self._tokens = self._host.tolist()
        return self._tokens


class Sampler:
    """Runs the sampling kernels over the logits rows a step returned."""

    def __init__(self, device):
        import torch
        self.device = device
        self._torch = torch

    def pick_async(self, logits, temperatures: Sequence[float], uniforms: Sequence[float]) -> PendingPick:
        """Queues the kernel and the copy of its result to the host; returns at once."""
        torch = self._torch
        from ..kernels import ops
        n = logits.shape[0]
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
        if all(t <= 0 for t in temperatures):
            ops.argmax_rows(logits, out)
        else:
            host = torch.tensor([list(temperatures), list(uniforms)], dtype=torch.float32, pin_memory=True)
            dev = host.to(logits.device, non_blocking=True)
            ops.sample_rows(logits, dev[0], dev[1], out)
        back = torch.empty(n, dtype=torch.int32, pin_memory=True)
        back.copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return PendingPick(out, back, event)

    def pick(self, logits, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        return self.pick_async(logits, temperatures, uniforms).tokens()
