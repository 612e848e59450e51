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
    waiting); `tokens()` waits for the copy to the host and returns them.
    The vectors are the sampler's own and are used again after `Sampler.RING`
    further picks: feed `on_device` to the next step or two, not later (the
    ids themselves are read out in time by the sampler if the caller has not)."""

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


class _PickBuffers:
    """What one pick needs, allocated once: the ids on the device and in pinned host memory,
    temperatures and uniform numbers in pinned host memory and on the device."""

    def __init__(self, torch, device, capacity: int):
        self.capacity = capacity
        self.ids = torch.empty(capacity, dtype=torch.int32, device=device)
        self.ids_host = torch.empty(capacity, dtype=torch.int32, pin_memory=True)
        self.params_host = torch.empty(2, capacity, dtype=torch.float32, pin_memory=True)
        self.params = torch.empty(2, capacity, dtype=torch.float32, device=device)
        self.last: Optional[PendingPick] = None


class Sampler:
    """Runs the sampling kernels over the logits rows a step returned. Its
    buffers go round in a ring, so a pick allocates nothing once the ring has
    seen the batch size."""
    RING = 8

    def __init__(self, device):
        import torch
        self.device = device
        self._torch = torch
        self._ring: List[Optional[_PickBuffers]] = [None] * self.RING
        self._turn = 0

    def _buffers(self, n: int) -> _PickBuffers:
        i = self._turn
        self._turn = (i + 1) % self.RING
        b = self._ring[i]
        if b is not None and b.last is not None:
            b.last.tokens()          # whoever still holds that pick finds its ids read out; the buffers are free
            b.last = None
        if b is None or b.capacity < n:
            b = self._ring[i] = _PickBuffers(self._torch, self.device, max(64, 1 << (n - 1).bit_length()))
        return b

    def pick_async(self, logits, temperatures: Sequence[float], uniforms: Sequence[float]) -> PendingPick:
        """Queues the kernel and the copy of its result to the host; returns at once."""
        torch = self._torch
        from ..kernels import ops
        n = logits.shape[0]
        b = self._buffers(n)
        out = b.ids[:n]
        if all(t <= 0 for t in temperatures):
            ops.argmax_rows(logits, out)
        else:
            b.params_host[0, :n] = torch.tensor(list(temperatures), dtype=torch.float32)
            b.params_host[1, :n] = torch.tensor(list(uniforms), dtype=torch.float32)
            b.params.copy_(b.params_host, non_blocking=True)
            ops.sample_rows(logits, b.params[0, :n], b.params[1, :n], out)
        back = b.ids_host[:n]
        back.copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        b.last = PendingPick(out, back, event)
        return b.last

    def pick(self, logits, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        return self.pick_async(logits, temperatures, uniforms).tokens()
