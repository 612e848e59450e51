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

import ctypes
import os
from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Tuple

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
    drawn: int = 0                   # tokens sampled for it that count, read back or not
    # while its last sampled token has not been read back:
    unread: bool = False
    ended_by_length: bool = False    # that token is its last; it has left the engine already
    repend: bool = False             # it was pre-empted meanwhile: `pending` lacks that token


@dataclass
class Planned:
    request: Request
    tokens: List[int]
    wants_logits: bool


class Scheduler:
    """`engine` needs: step(entries) -> logits rows or None, release(id),
    cache (a CacheManager), page_size. `pick(logits, temperatures, uniforms)`
    turns logits rows into token ids.

    The decisions (whom to admit, what each request feeds under the budget,
    whom to pre-empt) are taken by the native scheduler core
    (csrc/host/scheduler.cpp), which knows requests by size only; token
    values, sampling and the model step are handled here.

    With `pick_async` (logits, temperatures, uniforms -> an object with
    `on_device`, the int32 vector the tokens land in, and `tokens()`, which
    waits for them) the loop does not wait for a step's tokens before it
    queues the next step: a request's next token is fed from the device, the
    host reads it one step late, while the GPU is busy. Every sampled token is
    then counted as "goes on" at first; when it turns out to be a stop token
    the request is taken out (it has run one step in vain). What is generated
    is the same either way."""

    def __init__(self, engine, pick: Callable, max_batch_tokens: int = 2048, max_running: int = 64,
                 portion: Optional[int] = None, entry_type=None, pick_async: Optional[Callable] = None):
        from ..cache import native as N
        self._N = N
        self._lib = N.host_library()
        self.engine = engine
        self.pick = pick
        self.pick_async = pick_async
        self._unread = None              # (requests and their places, the pending pick) of the last step
        self.max_batch_tokens = max_batch_tokens
        self.max_running = max_running
        self.portion = portion or prefill_portion()
        self._s = self._lib.imparo_sched_new(engine.cache._c, max_batch_tokens, max_running, self.portion)
        if not self._s:
            raise ValueError("the scheduler refused its sizes")
        self._requests: Dict[int, Request] = {}          # by native handle: waiting or running
        self.finished: Dict[Hashable, Request] = {}
        self._arrivals = 0
        if entry_type is None:
            from .engine import StepEntry
            entry_type = StepEntry
        self._entry = entry_type
        self.log: List[Tuple] = []      # decisions, for tests and --verbose
        cap = max(64, max_running + 8)
        self._cap = cap
        self._ids = (ctypes.c_int64 * cap)()
        self._offs = (ctypes.c_int32 * cap)()
        self._counts = (ctypes.c_int32 * cap)()
        self._wants = (ctypes.c_int32 * cap)()
        self._ev_ids = (ctypes.c_int64 * (4 * cap))()
        self._ev_kinds = (ctypes.c_int32 * (4 * cap))()
        self._n_ev = ctypes.c_int32(0)

    def __del__(self):
        if getattr(self, "_s", None):
            self._lib.imparo_sched_delete(self._s)
            self._s = None

    def warm(self, longest_context: int) -> int:
        """Has the engine capture, now, every decode step this scheduler can come to run: 1 to
        `max_running` single-token rows at every block-table width up to `longest_context` tokens.
        A shape that is first met while serving costs several steps' time; this moves that cost
        to the start. Returns the number of shapes captured (0 for an engine that captures none)."""
        warm = getattr(self.engine, "warm", None)
        if warm is None:
            return 0
        page = self.engine.page_size
        contexts = sorted({min(longest_context, pages * page) for pages in range(1, -(-longest_context // page) + 1)})
        return warm(range(1, self.max_running + 1), contexts)

    # ------------------------------------------------------------ intake
    def add(self, request_id: Hashable, prompt: Sequence[int], params: SamplingParams) -> Request:
        if len(prompt) == 0:
            raise ValueError("a request needs at least one prompt token")
        r = Request(request_id, list(prompt), params, pending=list(prompt), arrival=self._arrivals)
        self._arrivals += 1
        # a request the step function would refuse ends here, alone, instead of failing a step that
        # carries other requests (the reference answers such a request with an error of its own before
        # it reaches the engine, /root/reference/crates/imparo-server/src/main.rs:1981-1987)
        vocab = getattr(self.engine, "vocab_size", None)
        if vocab is not None:
            bad = next((t for t in r.prompt if isinstance(t, bool) or not isinstance(t, int) or not 0 <= t < vocab),
                       None)
            if bad is not None:
                self._finish(r, f"error: token id {bad!r} is outside the vocabulary of {vocab}")
                return r
        limit = getattr(self.engine, "max_position", None)
        if limit is not None and len(r.prompt) + max(params.max_tokens, 1) - 1 > limit:
            self._finish(r, f"error: {len(r.prompt)} prompt tokens and {params.max_tokens} new ones pass the "
                            f"model's {limit} positions")
            return r
        h = self.engine.cache.handle(request_id)
        rc = self._lib.imparo_sched_add(self._s, h, len(prompt), params.max_tokens)
        if rc == 1:
            self._finish(r, "length")
            return r
        if rc < 0:
            raise ValueError(f"request {request_id!r} is already queued")
        self._requests[h] = r
        return r

    def has_work(self) -> bool:
        return bool(self._lib.imparo_sched_n_waiting(self._s) or self._lib.imparo_sched_n_running(self._s)
                    or self._unread is not None)

    def _listed(self, fn) -> List[Request]:
        buf = (ctypes.c_int64 * max(1, len(self._requests)))()
        n = fn(self._s, buf, len(buf))
        return [self._requests[buf[i]] for i in range(max(n, 0))]

    @property
    def waiting(self) -> List[Request]:
        return self._listed(self._lib.imparo_sched_waiting)

    @property
    def running(self) -> List[Request]:
        return self._listed(self._lib.imparo_sched_running)

    # ------------------------------------------------------------ decisions
    def plan(self) -> List[Planned]:
        """Chooses this step's batch; admits and pre-empts as needed."""
        n = self._lib.imparo_sched_plan(self._s, self._ids, self._offs, self._counts, self._wants, self._cap,
                                        self._ev_ids, self._ev_kinds, 4 * self._cap, ctypes.byref(self._n_ev))
        if n < 0:
            raise RuntimeError(f"the scheduler could not plan a step (code {n})")
        N = self._N
        for i in range(min(self._n_ev.value, 4 * self._cap)):
            h, kind = self._ev_ids[i], self._ev_kinds[i]
            r = self._requests[h]
            if kind == N.EV_ADMIT:
                self.log.append(("admit", r.id))
            elif kind == N.EV_WAIT:
                self.log.append(("wait", r.id))
            elif kind == N.EV_PREEMPT:
                # it gave back everything it held; it will recompute prompt ++ generated
                self.engine.release(r.id)
                r.pending = r.prompt + r.generated
                r.repend = r.unread            # its latest token joins `pending` when it has been read
                r.fed = 0
                r.next_token = None
                r.preemptions += 1
                self.log.append(("preempt", r.id))
            elif kind == N.EV_FAIL:
                self.engine.release(r.id)
                del self._requests[h]
                self._finish(r, "error: the request does not fit the cache even alone")
        planned = []
        for i in range(n):
            r = self._requests[self._ids[i]]
            off, count = self._offs[i], self._counts[i]
            tokens = [r.next_token] if off < 0 else r.pending[off:off + count]
            planned.append(Planned(r, tokens, bool(self._wants[i])))
        return planned

    def _finish(self, r: Request, reason: str) -> None:
        r.finished = True
        r.finish_reason = reason
        self.finished[r.id] = r
        self.engine.cache.forget(r.id)
        self.log.append(("finish", r.id, reason))

    # ------------------------------------------------------------ one iteration
    def step(self) -> List[Tuple[Hashable, int]]:
        """Plans, runs one engine step, samples. Returns (request, token) for
        every token handed out in this iteration."""
        planned = self.plan()
        if not planned:
            return self._read_back()
        entries = [self._entry(p.request.id, p.tokens, [len(p.tokens) - 1] if p.wants_logits else [])
                   for p in planned]
        logits = self.engine.step(entries)
        self._lib.imparo_sched_advance(self._s)
        for p in planned:
            r = p.request
            if r.fed < len(r.pending):
                r.fed += len(p.tokens)
            else:
                r.next_token = None           # the decoded token is in the cache now
        askers = [p.request for p in planned if p.wants_logits]
        if not askers:
            return self._read_back()
        temps = [r.params.temperature for r in askers]
        unis = [uniform_for(r.params.seed, r.drawn) for r in askers]
        if self.pick_async is not None:
            pending = self.pick_async(logits, temps, unis)
            out = self._read_back()          # the step before's tokens, while this step runs
            self._count_unread(askers, pending)
            return out
        out: List[Tuple[Hashable, int]] = []
        picks = self.pick(logits, temps, unis)
        for r, tok in zip(askers, picks):
            tok = int(tok)
            h = self.engine.cache.handle(r.id)
            is_stop = tok in r.params.stop_token_ids      # a stop token ends the reply unsent
            outcome = self._lib.imparo_sched_token(self._s, h, int(is_stop))
            if not is_stop:
                r.drawn += 1
                r.generated.append(tok)
                out.append((r.id, tok))
            if outcome == 0:
                r.next_token = tok
            else:                                          # 1: stop; 2: the last token needs no forward
                self.engine.release(r.id)
                del self._requests[h]
                self._finish(r, "stop" if outcome == 1 else "length")
        return out

    def _count_unread(self, askers: List[Request], pending) -> None:
        """Counts tokens that were asked for but not read yet, as tokens after which the reply goes on."""
        from .engine import DeviceToken
        places = []
        for i, r in enumerate(askers):
            if r.finished:                     # a late stop token ended it while this step ran
                continue
            h = self.engine.cache.handle(r.id)
            outcome = self._lib.imparo_sched_token(self._s, h, 0)
            r.drawn += 1
            r.unread = True
            if outcome == 0:
                r.next_token = DeviceToken(pending.on_device, i)
            else:                              # 2: its last token; it needs no forward and leaves the engine now
                self.engine.release(r.id)
                del self._requests[h]
                r.ended_by_length = True
            places.append((r, i))
        self._unread = (places, pending)

    def _read_back(self) -> List[Tuple[Hashable, int]]:
        """Waits for the tokens of the step before and hands them out."""
        if self._unread is None:
            return []
        places, pending = self._unread
        self._unread = None
        tokens = pending.tokens()
        out: List[Tuple[Hashable, int]] = []
        for r, i in places:
            tok = int(tokens[i])
            r.unread = False
            is_stop = tok in r.params.stop_token_ids
            if r.finished:                                 # it failed meanwhile: the token still counts
                if not is_stop:
                    r.generated.append(tok)
                    out.append((r.id, tok))
                continue
            if is_stop:                                    # ends the reply unsent, one step late
                if not r.ended_by_length:
                    h = self.engine.cache.handle(r.id)
                    self._lib.imparo_sched_retract(self._s, h)
                    self.engine.release(r.id)
                    self._requests.pop(h, None)
                self._finish(r, "stop")
                continue
            r.generated.append(tok)
            out.append((r.id, tok))
            if r.ended_by_length:
                self._finish(r, "length")
                continue
            if r.next_token is not None and not isinstance(r.next_token, int):
                r.next_token = tok                         # not fed yet: the host's copy will do
            if r.repend:
                r.pending = r.prompt + r.generated
                r.repend = False
        return out

    def run(self) -> Dict[Hashable, Request]:
        while self.has_work():
            n_running = self._lib.imparo_sched_n_running(self._s)
            before = (self._lib.imparo_sched_n_waiting(self._s), n_running, len(self.finished))
            self.step()
            after = (self._lib.imparo_sched_n_waiting(self._s), self._lib.imparo_sched_n_running(self._s),
                     len(self.finished))
            if after[1] == 0 and after[0] and before == after and n_running == 0 and self._unread is None:
                head = ctypes.c_int64(0)                       # nothing runs and the head still cannot start
                if self._lib.imparo_sched_drop_waiting_head(self._s, ctypes.byref(head)):
                    r = self._requests.pop(head.value)
                    self._finish(r, "error: the request does not fit the cache even alone")
        return self.finished


def generate(model, input_ids: Sequence[Sequence[int]], max_tokens: int = 16, temperature: float = 0.0,
             seed: int = 0, stop_token_ids: Optional[Sequence[int]] = None, dtype: str = "bfloat16",
             ctx: Optional[int] = None, parallel: int = 64, max_batch_tokens: int = 2048,
             page_size: int = 64, overlap: bool = True, num_pages=None,
             kv_budget_bytes: Optional[int] = None) -> List[List[int]]:
    """Tokens in, tokens out. `model` is a model folder or an Engine; returns
    the generated ids of every prompt, in order. Request `i` samples with seed
    `seed + i`. `ctx` is the most tokens one request may hold (the reference's
    -c/--ctx), `parallel` the most requests that run at once (-np/--parallel).
    `overlap`: queue each step before the tokens of the step before are read
    back (the same tokens come out; False waits after every step).
    `num_pages` or `kv_budget_bytes` size the cache pools instead of `ctx` and
    `parallel` (a smaller pool makes requests wait or be recomputed)."""
    from .engine import Engine
    from ..sampling.sampler import Sampler
    if len(input_ids) == 0:
        return []
    if isinstance(model, Engine):
        engine = model
    else:
        longest = max(len(p) for p in input_ids) + max_tokens
        per_request = ctx or longest
        n_live = min(parallel, len(input_ids))
        rounded = ((per_request + page_size - 1) // page_size + 1) * page_size
        sized = num_pages is not None or kv_budget_bytes is not None
        engine = Engine(model, dtype=dtype, max_tokens=None if sized else rounded * n_live, page_size=page_size,
                        max_requests=max(1, n_live), num_pages=num_pages, kv_budget_bytes=kv_budget_bytes,
                        max_step_tokens=max(max_batch_tokens, 1))
    stops = tuple(stop_token_ids) if stop_token_ids is not None else tuple(engine.plan.stop_token_ids)
    sampler = Sampler(engine.device)
    sched = Scheduler(engine, sampler.pick, max_batch_tokens=max_batch_tokens,
                      max_running=min(parallel, engine.cache.n_slots),
                      pick_async=sampler.pick_async if overlap else None)
    for i, prompt in enumerate(input_ids):
        sched.add(i, prompt, SamplingParams(temperature=temperature, max_tokens=max_tokens, seed=seed + i,
                                            stop_token_ids=stops))
        if sched.finished.get(i) is not None and sched.finished[i].finish_reason.startswith("error"):
            raise ValueError(f"request {i}: {sched.finished[i].finish_reason[7:]}")
    done = sched.run()
    for i in range(len(input_ids)):
        if done[i].finish_reason.startswith("error"):
            raise RuntimeError(f"request {i}: {done[i].finish_reason}")
    return [done[i].generated for i in range(len(input_ids))]
