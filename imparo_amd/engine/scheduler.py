"""Continuous batching above the step function.

One loop iteration: take new requests in arrival order while they fit, give
every running request its next tokens under a token budget (one decoded token
each first, then portions of prompts), run ONE step with all of them, hand out
the sampled tokens, finish and free. The reference's loop has the same order
of duties but runs a newcomer's chunk as a forward of its own
(/root/reference/crates/imparo-server/src/sched.rs:4-19,286-310).

When pages run out the youngest running request is pre-empted: it gives back
its pages and its slot and returns to the head of the waiting line with
prompt ++ generated as its new prompt, to be recomputed. (The reference parks
such a row on a disk tier, sched.rs:483-488,701-732; there is none here.) A
request that cannot fit even alone ends with an error.
"""
from __future__ import annotations

import os
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..cache.pages import OutOfPages
from ..sampling.sampler import SamplingParams, uniform_for

DEFAULT_PORTION = 512   # the reference's prefill chunk (crates/imparo-model/src/lib.rs:1000)


def prefill_portion() -> int:
    """Tokens of one prompt per step; IMPARO_BATCH overrides, as in the
    reference (crates/imparo-model/src/lib.rs:1008-1014)."""
    try:
        v = int(os.environ.get("IMPARO_BATCH", DEFAULT_PORTION))
        return v if v > 0 else DEFAULT_PORTION
    except ValueError:
        return DEFAULT_PORTION


@dataclass
class Request:
    id: Hashable
    prompt: List[int]
    params: SamplingParams
    generated: List[int] = field(default_factory=list)
    # tokens to (re)compute before decoding goes on: the prompt, plus what was
    # generated before a pre-emption
    pending: List[int] = field(default_factory=list)
    fed: int = 0                     # how many of `pending` the cache holds
    next_token: Optional[int] = None  # sampled, not yet fed
    finished: bool = False
    finish_reason: str = ""
    preemptions: int = 0
    arrival: int = 0


@dataclass
class Planned:
    request: Request
    tokens: List[int]
    wants_logits: bool


class Scheduler:
    """`engine` needs: step(entries) -> logits rows or None, release(id),
    cache (a CacheManager), page_size. `pick(logits, temperatures, uniforms)`
    turns logits rows into token ids."""

    def __init__(self, engine, pick: Callable, max_batch_tokens: int = 2048, max_running: int = 64,
                 portion: Optional[int] = None, entry_type=None):
        self.engine = engine
        self.pick = pick
        self.max_batch_tokens = max_batch_tokens
        self.max_running = max_running
        self.portion = portion or prefill_portion()
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: Dict[Hashable, Request] = {}
        self._arrivals = 0
        if entry_type is None:
            from .engine import StepEntry
            entry_type = StepEntry
        self._entry = entry_type
        self.log: List[Tuple] = []      # decisions, for tests and --verbose

    # ------------------------------------------------------------ intake
    def add(self, request_id: Hashable, prompt: Sequence[int], params: SamplingParams) -> Request:
        if len(prompt) == 0:
            raise ValueError("a request needs at least one prompt token")
        r = Request(request_id, list(prompt), params, pending=list(prompt), arrival=self._arrivals)
        self._arrivals += 1
        if params.max_tokens <= 0:
            self._finish(r, "length")
            return r
        self.waiting.append(r)
        return r

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------ decisions
    def _pages_for(self, n_tokens: int) -> int:
        ps = self.engine.page_size
        return (n_tokens + ps - 1) // ps

    def _free_pages(self) -> int:
        free = self.engine.cache.free_pages()
        return min(free) if free else 1 << 30

    def _next_tokens(self, r: Request, budget: int) -> Tuple[List[int], bool]:
        """What `r` would feed next under `budget` tokens, and whether that
        ends in a place whose logits are needed."""
        if r.fed < len(r.pending):
            n = min(self.portion, budget, len(r.pending) - r.fed)
            return r.pending[r.fed:r.fed + n], r.fed + n == len(r.pending) and r.next_token is None
        return [r.next_token], True

    def _pages_needed(self, p: Planned) -> int:
        cache = self.engine.cache
        if cache.is_live(p.request.id):
            need = cache.pages_needed(p.request.id, cache.length[p.request.id] + len(p.tokens))
            return max(need) if need else 0
        return self._pages_for(len(p.tokens))

    def plan(self) -> List[Planned]:
        """Chooses this step's batch; admits and pre-empts as needed."""
        budget = self.max_batch_tokens
        planned: List[Planned] = []
        # 1. running requests: decoders first, then prompts in progress
        order = sorted(self.running, key=lambda r: (r.fed < len(r.pending), r.arrival))
        for r in order:
            if budget <= 0:
                break
            toks, wants = self._next_tokens(r, budget)
            planned.append(Planned(r, toks, wants))
            budget -= len(toks)
        spoken_for = sum(self._pages_needed(p) for p in planned)
        # 2. admissions, first come first served; the head of the line blocks the rest.
        # A newcomer needs the pages of its first portion and leaves one page of
        # headroom per running request
        # (/root/reference/crates/imparo-server/src/main.rs:2230-2246).
        while self.waiting and budget > 0 and len(self.running) < self.max_running:
            r = self.waiting[0]
            toks, wants = self._next_tokens(r, budget)
            need = self._pages_for(len(toks)) + len(self.running)
            if self.engine.cache.slots.n_free == 0 or (self.running and need > self._free_pages() - spoken_for):
                self.log.append(("wait", r.id))
                break
            self.waiting.popleft()
            self.running.append(r)
            self.log.append(("admit", r.id))
            planned.append(Planned(r, toks, wants))
            spoken_for += self._pages_for(len(toks))
            budget -= len(toks)
        # 3. do the pages suffice? if not, the youngest running request goes back in line
        while planned:
            if sum(self._pages_needed(p) for p in planned) <= self._free_pages():
                break
            if len(self.running) == 1:
                r = self.running[0]
                self._leave(r)
                self._finish(r, "error: the request does not fit the cache even alone")
                planned = []
                break
            victim = max(self.running, key=lambda r: r.arrival)
            self.preempt(victim)
            planned = [p for p in planned if p.request is not victim]
        return planned

    def preempt(self, r: Request) -> None:
        """Gives back everything `r` holds; it will recompute prompt ++ generated."""
        self._leave(r)
        r.pending = r.prompt + r.generated
        r.fed = 0
        r.next_token = None
        r.preemptions += 1
        self.waiting.appendleft(r)
        self.log.append(("preempt", r.id))

    def _leave(self, r: Request) -> None:
        if r in self.running:
            self.running.remove(r)
        self.engine.release(r.id)

    def _finish(self, r: Request, reason: str) -> None:
        r.finished = True
        r.finish_reason = reason
        self.finished[r.id] = r
        self.log.append(("finish", r.id, reason))

    # ------------------------------------------------------------ one iteration
    def step(self) -> List[Tuple[Hashable, int]]:
        """Plans, runs one engine step, samples. Returns (request, token) for
        every token handed out in this iteration."""
        planned = self.plan()
        if not planned:
            return []
        entries = [self._entry(p.request.id, p.tokens, [len(p.tokens) - 1] if p.wants_logits else [])
                   for p in planned]
        logits = self.engine.step(entries)
        for p in planned:
            r = p.request
            if r.fed < len(r.pending):
                r.fed += len(p.tokens)
            else:
                r.next_token = None           # the decoded token is in the cache now
        askers = [p.request for p in planned if p.wants_logits]
        out: List[Tuple[Hashable, int]] = []
        if askers:
            temps = [r.params.temperature for r in askers]
            unis = [uniform_for(r.params.seed, len(r.generated)) for r in askers]
            picks = self.pick(logits, temps, unis)
            for r, tok in zip(askers, picks):
                tok = int(tok)
                if tok in r.params.stop_token_ids:     # a stop token ends the reply unsent
                    self._leave(r)
                    self._finish(r, "stop")
                    continue
                r.generated.append(tok)
                out.append((r.id, tok))
                if len(r.generated) >= r.params.max_tokens:   # the last token needs no forward
                    self._leave(r)
                    self._finish(r, "length")
                else:
                    r.next_token = tok
        return out

    def run(self) -> Dict[Hashable, Request]:
        while self.has_work():
            before = (len(self.waiting), len(self.running), len(self.finished))
            self.step()
            if not self.running and self.waiting and before == (len(self.waiting), 0, len(self.finished)):
                r = self.waiting.popleft()      # nothing runs and the head still cannot start
                self._finish(r, "error: the request does not fit the cache even alone")
        return self.finished


def generate(model, input_ids: Sequence[Sequence[int]], max_tokens: int = 16, temperature: float = 0.0,
             seed: int = 0, stop_token_ids: Optional[Sequence[int]] = None, dtype: str = "bfloat16",
             ctx: Optional[int] = None, parallel: int = 64, max_batch_tokens: int = 2048,
             page_size: int = 64) -> List[List[int]]:
    """Tokens in, tokens out. `model` is a model folder or an Engine; returns
    the generated ids of every prompt, in order. Request `i` samples with seed
    `seed + i`. `ctx` is the most tokens one request may hold (the reference's
    -c/--ctx), `parallel` the most requests that run at once (-np/--parallel)."""
    from .engine import Engine
    from ..sampling.sampler import Sampler
    if isinstance(model, Engine):
        engine = model
    else:
        longest = max(len(p) for p in input_ids) + max_tokens
        per_request = ctx or longest
        n_live = min(parallel, len(input_ids))
        rounded = ((per_request + page_size - 1) // page_size + 1) * page_size
        engine = Engine(model, dtype=dtype, max_tokens=rounded * n_live, page_size=page_size,
                        max_requests=max(1, n_live))
    stops = tuple(stop_token_ids) if stop_token_ids is not None else tuple(engine.plan.stop_token_ids)
    sampler = Sampler(engine.device)
    sched = Scheduler(engine, sampler.pick, max_batch_tokens=max_batch_tokens,
                      max_running=min(parallel, engine.cache.n_slots))
    for i, prompt in enumerate(input_ids):
        sched.add(i, prompt, SamplingParams(temperature=temperature, max_tokens=max_tokens, seed=seed + i,
                                            stop_token_ids=stops))
    done = sched.run()
    for i in range(len(input_ids)):
        if done[i].finish_reason.startswith("error"):
            raise RuntimeError(f"request {i}: {done[i].finish_reason}")
    return [done[i].generated for i in range(len(input_ids))]
