"""The scheduler's decisions, on the host, with the real cache manager and a
stand-in for the model: admission in arrival order, portions under a token
budget, decoding, finishing and freeing, and what happens when pages run out."""
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import pytest

from imparo_amd.cache import CacheManager, kv_spec, FixedSpec, OutOfPages
from imparo_amd.engine.engine import DeviceToken
from imparo_amd.engine.scheduler import Scheduler, Request
from imparo_amd.sampling import SamplingParams, uniform_for

VOCAB = 50


@dataclass
class Entry:
    request: object
    tokens: Sequence[int]
    want: Sequence[int] = ()


class FakeEngine:
    """Keeps the tokens each live request has fed and answers with logits that
    are a pure function of that history; pages and slots are the real thing."""

    def __init__(self, n_pages, page_size=4, n_slots=4):
        self.page_size = page_size
        self.cache = CacheManager([kv_spec(1, 16), FixedSpec((2, 4))], page_size, n_pages, n_slots)
        self.history = {}
        self.steps = []          # [(request, n_tokens, wants)] per step

    @staticmethod
    def next_of(history: List[int]) -> int:
        h = 7
        for i, t in enumerate(history):
            h = (h * 31 + (t + 1) * (i + 3)) % 1000003
        return h % VOCAB

    def step(self, entries):
        taken = []
        try:
            for e in entries:
                if not self.cache.is_live(e.request):
                    self.cache.admit(e.request)
                    self.history[e.request] = []
                taken.append((e.request, self.cache.reserve(e.request, self.cache.length[e.request] + len(e.tokens))))
        except OutOfPages:
            raise AssertionError("the scheduler sent a step that does not fit")
        rows = []
        for e in entries:
            # a token that "is still on the device" is looked up where the fake sampler left it
            e.tokens = [t.source[t.index] if isinstance(t, DeviceToken) else t for t in e.tokens]
            self.history[e.request].extend(e.tokens)
            self.cache.commit(e.request, len(self.history[e.request]))
            for w in e.want:
                assert w == len(e.tokens) - 1
                row = np.zeros(VOCAB, dtype=np.float32)
                row[self.next_of(self.history[e.request])] = 1.0
                rows.append(row)
        self.steps.append([(e.request, len(e.tokens), bool(e.want)) for e in entries])
        self.cache.check()
        return np.stack(rows) if rows else None

    def release(self, request):
        if self.cache.is_live(request):
            self.cache.release(request)
            del self.history[request]


def pick(logits, temperatures, uniforms):
    return [int(np.argmax(r)) for r in logits]


def expected(prompt, n):
    seq, out = list(prompt), []
    for _ in range(n):
        t = FakeEngine.next_of(seq)
        out.append(t)
        seq.append(t)
    return out


class FakePending:
    """What an asynchronous sampler hands back: the tokens "on the device", and a wait for them."""
    reads = 0

    def __init__(self, tokens):
        self.on_device = tokens

    def tokens(self):
        FakePending.reads += 1
        return self.on_device


def pick_async(logits, temperatures, uniforms):
    return FakePending(pick(logits, temperatures, uniforms))


def make(n_pages=64, overlap=False, **kw):
    eng = FakeEngine(n_pages)
    return eng, Scheduler(eng, pick, entry_type=Entry, pick_async=pick_async if overlap else None, **kw)


def test_one_request_prompt_in_portions_then_decode():
    eng, s = make(max_batch_tokens=8, portion=5)
    s.add("a", list(range(12)), SamplingParams(max_tokens=4))
    done = s.run()
    assert done["a"].generated == expected(range(12), 4) and done["a"].finish_reason == "length"
    # 12 tokens in portions of 5: 5, 5, 2 (logits only after the last), then 3 decode steps:
    # the last token needs no forward
    assert eng.steps == [[("a", 5, False)], [("a", 5, False)], [("a", 2, True)],
                         [("a", 1, True)], [("a", 1, True)], [("a", 1, True)]]
    assert eng.cache.free_pages() == [64] and eng.cache.slots.n_free == 4


def test_decodes_ride_with_portions_under_the_budget():
    eng, s = make(max_batch_tokens=8, portion=6)
    s.add("a", [1, 2, 3], SamplingParams(max_tokens=6))
    s.step()                         # a's prompt, first token sampled
    s.add("b", list(range(20)), SamplingParams(max_tokens=2))
    s.step()
    # a decodes (1 token) and b's first portion takes what the budget leaves, at most a portion
    assert eng.steps[-1] == [("a", 1, True), ("b", 6, False)]
    s.step()
    assert eng.steps[-1] == [("a", 1, True), ("b", 6, False)]
    done = s.run()
    assert done["a"].generated == expected([1, 2, 3], 6) and done["b"].generated == expected(range(20), 2)
    assert all(sum(n for _, n, _ in st) <= 8 for st in eng.steps)


def test_arrival_order_and_running_cap():
    eng, s = make(max_batch_tokens=64, max_running=2)
    for name in "abc":
        s.add(name, [ord(name)] * 3, SamplingParams(max_tokens=3))
    s.step()
    assert [r.id for r in s.running] == ["a", "b"] and [r.id for r in s.waiting] == ["c"]
    done = s.run()
    assert [e for e in s.log if e[0] == "admit"] == [("admit", "a"), ("admit", "b"), ("admit", "c")]
    assert all(done[n].generated == expected([ord(n)] * 3, 3) for n in "abc")


def test_newcomers_of_one_step_do_not_share_a_slot():
    eng = FakeEngine(64, n_slots=2)
    s = Scheduler(eng, pick, entry_type=Entry, max_batch_tokens=64, max_running=8)
    for name in "abc":
        s.add(name, [ord(name)] * 3, SamplingParams(max_tokens=2))
    s.step()
    assert [r.id for r in s.running] == ["a", "b"] and [r.id for r in s.waiting] == ["c"]
    done = s.run()
    assert all(done[n].generated == expected([ord(n)] * 3, 2) for n in "abc")
    assert eng.cache.slots.n_free == 2


def test_stop_token_ends_the_reply_unsent():
    want = expected([5, 6], 5)
    eng, s = make()
    s.add("a", [5, 6], SamplingParams(max_tokens=5, stop_token_ids=(want[2],)))
    done = s.run()
    assert done["a"].generated == want[:2] and done["a"].finish_reason == "stop"
    assert eng.cache.free_pages() == [64]


def test_zero_max_tokens_runs_nothing():
    eng, s = make()
    s.add("a", [1], SamplingParams(max_tokens=0))
    assert s.run()["a"].generated == [] and eng.steps == []


def test_a_request_the_step_function_would_refuse_ends_alone():
    """A token outside the vocabulary, or a reply that would pass the model's
    positions, ends that request with an error when it is added; the others run
    as if it had never come and nothing of it is left in the cache."""
    eng, s = make()
    eng.vocab_size, eng.max_position = VOCAB, 40
    s.add("good", [1, 2, 3], SamplingParams(max_tokens=5))
    bad = s.add("bad id", [1, VOCAB, 3], SamplingParams(max_tokens=5))
    long = s.add("too long", list(range(30)), SamplingParams(max_tokens=12))
    fits = s.add("just fits", list(range(30)), SamplingParams(max_tokens=11))
    assert bad.finished and "outside the vocabulary" in bad.finish_reason
    assert long.finished and "positions" in long.finish_reason and not fits.finished
    done = s.run()
    assert done["good"].generated == expected([1, 2, 3], 5)
    assert done["just fits"].generated == expected(list(range(30)), 11)
    assert all(kind != "bad id" and kind != "too long" for step in eng.steps for kind, _, _ in step)
    assert not eng.history and eng.cache.slots.n_free == eng.cache.n_slots
    eng.cache.check()


def test_waits_at_the_head_of_the_line_until_pages_free_up():
    # 6 pages of 4: a (prompt 12 -> 3 pages) runs; b needs 3 pages + 1 of headroom for a: waits
    eng, s = make(n_pages=6, max_batch_tokens=64, portion=64)
    s.add("a", list(range(12)), SamplingParams(max_tokens=3))
    s.add("b", list(range(12)), SamplingParams(max_tokens=2))
    s.add("c", [1], SamplingParams(max_tokens=2))
    s.step()
    assert [r.id for r in s.running] == ["a"]
    assert ("wait", "b") in s.log and ("admit", "c") not in s.log     # c does not jump the line
    done = s.run()
    assert done["b"].generated == expected(range(12), 2) and done["c"].generated == expected([1], 2)


def test_out_of_pages_preempts_the_youngest_and_outputs_do_not_change():
    # 5 pages of 4 = 20 positions; two requests that grow to 14 each cannot both stay
    eng, s = make(n_pages=5, max_batch_tokens=64, portion=64)
    s.add("old", list(range(6)), SamplingParams(max_tokens=8))
    s.add("young", list(range(10, 16)), SamplingParams(max_tokens=8))
    done = s.run()
    assert ("preempt", "young") in s.log and ("preempt", "old") not in s.log
    assert done["old"].generated == expected(range(6), 8)
    assert done["young"].generated == expected(range(10, 16), 8)
    assert done["young"].preemptions >= 1 and done["old"].preemptions == 0
    # the pre-empted request came back with prompt ++ generated as its prompt
    refeeds = [st for st in eng.steps if any(r == "young" and n > 6 for r, n, _ in st)]
    assert refeeds
    assert eng.cache.free_pages() == [5] and eng.cache.slots.n_free == 4


def test_a_request_that_cannot_fit_alone_ends_with_an_error():
    eng, s = make(n_pages=2, max_batch_tokens=64, portion=64)
    s.add("big", list(range(9)), SamplingParams(max_tokens=2))
    s.add("ok", [1, 2], SamplingParams(max_tokens=2))
    done = s.run()
    assert done["big"].finish_reason.startswith("error") and done["big"].generated == []
    assert done["ok"].generated == expected([1, 2], 2)
    # and one that outgrows the pool while decoding alone
    eng, s = make(n_pages=2, max_batch_tokens=64, portion=64)
    s.add("grow", list(range(7)), SamplingParams(max_tokens=5))
    done = s.run()
    assert done["grow"].finish_reason.startswith("error") and done["grow"].generated == expected(range(7), 2)
    assert eng.cache.free_pages() == [2]


@pytest.mark.parametrize("seed", range(4))
def test_random_workloads_finish_with_the_right_tokens_and_give_everything_back(seed):
    rng = np.random.default_rng(seed)
    eng, s = make(n_pages=14, max_batch_tokens=24, portion=7, max_running=3)
    want = {}
    pending = []
    for i in range(10):
        prompt = rng.integers(0, VOCAB, size=int(rng.integers(1, 20))).tolist()
        n = int(rng.integers(1, 12))
        pending.append((i, prompt, n))
        want[i] = expected(prompt, n)
    # arrivals in waves
    while pending or s.has_work():
        for _ in range(int(rng.integers(0, 3))):
            if pending:
                i, prompt, n = pending.pop(0)
                s.add(i, prompt, SamplingParams(max_tokens=n))
        if s.has_work():
            s.step()
            assert sum(n for _, n, _ in eng.steps[-1]) <= 24 if eng.steps else True
            assert len(s.running) <= 3
    for i in want:
        assert s.finished[i].generated == want[i], (i, s.finished[i].finish_reason)
    assert eng.cache.free_pages() == [14] and eng.cache.slots.n_free == 4


def test_uniform_numbers_depend_on_seed_and_index_only():
    a = [uniform_for(3, i) for i in range(100)]
    assert a == [uniform_for(3, i) for i in range(100)]
    assert all(0.0 <= u < 1.0 for u in a) and len(set(a)) > 90
    assert a != [uniform_for(4, i) for i in range(100)]
    assert 0.35 < sum(a) / 100 < 0.65


# ---------------------------------------------------------------- the next step queued before the tokens are read
def test_overlapped_steps_feed_tokens_from_the_device_and_read_them_a_step_late():
    eng, s = make(overlap=True, max_batch_tokens=8, portion=5)
    s.add("a", list(range(12)), SamplingParams(max_tokens=4))
    assert s.step() == [] and s.step() == [] and s.step() == []     # the prompt; its token is not read yet
    want = expected(range(12), 4)
    assert s.step() == [("a", want[0])]          # the first decode step is queued, then token 0 is read
    assert s.step() == [("a", want[1])]
    assert s.step() == [("a", want[2])]          # the third decode step; a's last token needs no forward
    assert eng.cache.free_pages() == [64] and s.has_work()          # it left the engine; its token is unread
    assert s.step() == [("a", want[3])] and not s.has_work()
    assert s.finished["a"].generated == want and s.finished["a"].finish_reason == "length"
    assert eng.steps == [[("a", 5, False)], [("a", 5, False)], [("a", 2, True)],
                         [("a", 1, True)], [("a", 1, True)], [("a", 1, True)]]


def test_a_late_stop_token_costs_one_step_and_changes_nothing_else():
    want = expected([5, 6], 5)
    eng, s = make(overlap=True)
    s.add("a", [5, 6], SamplingParams(max_tokens=5, stop_token_ids=(want[2],)))
    done = s.run()
    assert done["a"].generated == want[:2] and done["a"].finish_reason == "stop"
    assert len(eng.steps) == 4                   # prompt, two decodes, and one in vain (3 without overlap)
    assert eng.cache.free_pages() == [64] and eng.cache.slots.n_free == 4
    # a stop token as the last token allowed: the reason is the stop, the token stays unsent
    eng, s = make(overlap=True)
    s.add("a", [5, 6], SamplingParams(max_tokens=3, stop_token_ids=(want[2],)))
    done = s.run()
    assert done["a"].generated == want[:2] and done["a"].finish_reason == "stop"


@pytest.mark.parametrize("seed", range(6))
def test_overlapped_and_waiting_loops_generate_the_same(seed):
    """Random arrivals, stop tokens, so few pages that requests are pre-empted and some fail."""
    runs = []
    for overlap in (False, True):
        rng = np.random.default_rng(seed)
        eng, s = make(n_pages=12, overlap=overlap, max_batch_tokens=24, portion=7, max_running=3)
        pending = []
        for i in range(12):
            prompt = rng.integers(0, VOCAB, size=int(rng.integers(1, 20))).tolist()
            n = int(rng.integers(1, 14))
            stops = tuple(rng.integers(0, VOCAB, size=int(rng.integers(0, 6))).tolist())
            pending.append((i, prompt, n, stops))
        while pending or s.has_work():
            for _ in range(int(rng.integers(0, 3))):
                if pending:
                    i, prompt, n, stops = pending.pop(0)
                    s.add(i, prompt, SamplingParams(max_tokens=n, stop_token_ids=stops))
            if s.has_work():
                s.step()
                assert len(s.running) <= 3
        assert eng.cache.free_pages() == [12] and eng.cache.slots.n_free == 4
        runs.append({i: (r.generated, r.finish_reason) for i, r in s.finished.items()})
        # against the plain recurrence
        rng = np.random.default_rng(seed)
        for i in range(12):
            prompt = rng.integers(0, VOCAB, size=int(rng.integers(1, 20))).tolist()
            n = int(rng.integers(1, 14))
            stops = tuple(rng.integers(0, VOCAB, size=int(rng.integers(0, 6))).tolist())
            got, reason = runs[-1][i]
            if reason.startswith("error"):
                continue
            full = expected(prompt, n)
            cut = next((j for j, t in enumerate(full) if t in stops), None)
            assert got == (full if cut is None else full[:cut]) and reason == ("length" if cut is None else "stop")
    assert runs[0] == runs[1]
    assert any(len(g) for g, _ in runs[0].values())


def test_overlapped_preemption_keeps_the_unread_token():
    eng, s = make(n_pages=5, overlap=True, max_batch_tokens=64, portion=64)
    s.add("old", list(range(6)), SamplingParams(max_tokens=8))
    s.add("young", list(range(10, 16)), SamplingParams(max_tokens=8))
    done = s.run()
    assert ("preempt", "young") in s.log
    assert done["old"].generated == expected(range(6), 8)
    assert done["young"].generated == expected(range(10, 16), 8)
    assert eng.cache.free_pages() == [5] and eng.cache.slots.n_free == 4
