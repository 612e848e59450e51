"""The engine against the plain implementation, in float32 and in bfloat16:
each request alone and whole; most of it in one step and the last 32 tokens one
by one; portions of changing size down to two tokens; mixed batches of up to
four live requests with so few pages that they are used again; long decoding;
the first tokens of a sequence. Variants with sharpened attention make a
single wrong or missing key visible, which random weights would average away.
"""
import os
import random

import pytest
import torch

from conftest import prompt_tokens
from gpu_helpers import make_engine, mixed_schedule, peak_pages, RefCache, step_all
from tolerances import check_logits

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
# (model, dtype): the sharpened models run in float32 only, the keen ones in both
CASES = [(m, d) for m in ("A", "B", "C", "A_keen", "C_keen") for d in DTYPES] + \
        [("A_sharp", "float32"), ("C_sharp", "float32")]


@pytest.fixture(scope="module")
def zoo(model_dirs, tmp_path_factory):
    """Model folders (with the sharpened variants), plain models, reference caches."""
    from safetensors.torch import load_file
    from imparo_amd.weights import save_file
    from plain_lfm2 import PlainLfm2
    import json, shutil
    dirs = dict(model_dirs)
    for base, tag, factor in (("A", "sharp", 3.0), ("C", "sharp", 3.0), ("A", "keen", 1.5), ("C", "keen", 1.5)):
        d = str(tmp_path_factory.mktemp(f"tiny_{base}_{tag}"))
        shutil.copy(os.path.join(model_dirs[base], "config.json"), d)
        t = load_file(os.path.join(model_dirs[base], "model.safetensors"))
        for k in list(t):
            # scores scale with |q||k|: with both norms times 3 their spread is 9 instead of 1 and the
            # softmax picks out single keys ("sharp", float32 only); times 1.5 it is 2.25 ("keen"), which
            # bfloat16 can still follow: a score of size s carries a rounding of s * 2^-8 from q and k,
            # and the sharp models turn that into weight shifts of several percent -- conditioning, not a fault
            if k.endswith("q_layernorm.weight") or k.endswith("k_layernorm.weight"):
                t[k] = (t[k].float() * factor).to(t[k].dtype)
        save_file(t, os.path.join(d, "model.safetensors"))
        dirs[f"{base}_{tag}"] = d
    plains = {k: PlainLfm2(v) for k, v in dirs.items()}
    return dirs, {k: RefCache(p) for k, p in plains.items()}


@pytest.fixture(scope="module")
def engines(zoo):
    cache = {}

    def get(name, dtype, **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in cache:
            cache[key] = make_engine(zoo[0][name], dtype, **kw)
        return cache[key]
    return get


def vocab_of(zoo, name):
    return zoo[1][name].plain.cfg["vocab_size"]


@pytest.mark.parametrize("name,dtype", CASES)
def test_each_request_alone_and_whole(zoo, engines, name, dtype):
    eng = engines(name, dtype)
    for n, seed in ((5, 1), (17, 2), (31, 3), (150, 4)):
        toks = prompt_tokens(vocab_of(zoo, name), n, seed)
        got = step_all(eng, "w", toks, [n])
        eng.release("w")
        check_logits(got, zoo[1][name](toks), dtype, f"{name} whole {n}")


@pytest.mark.parametrize("name,dtype", CASES)
def test_last_32_tokens_one_by_one(zoo, engines, name, dtype):
    eng = engines(name, dtype)
    toks = prompt_tokens(vocab_of(zoo, name), 150, 4)
    got = step_all(eng, "s", toks, [118] + [1] * 32)
    eng.release("s")
    check_logits(got, zoo[1][name](toks), dtype, f"{name} stepwise")


@pytest.mark.parametrize("name,dtype", CASES)
def test_portions_of_changing_size(zoo, engines, name, dtype):
    eng = engines(name, dtype)
    toks = prompt_tokens(vocab_of(zoo, name), 150, 4)
    ref, rel = zoo[1][name](toks), None
    for cuts in ([2, 3, 7, 2, 16, 5, 33, 2, 1, 64], [4], [7], [2], [63, 1, 2, 17]):
        got = step_all(eng, "p", toks, cuts)
        eng.release("p")
        check_logits(got, ref, dtype, f"{name} portions {cuts}", rel)


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_with_pages_used_again(zoo, engines, name, dtype):
    from imparo_amd.engine import StepEntry
    rng = random.Random(11)
    lengths = [70, 33, 121, 9, 64, 50, 97, 18]
    V = vocab_of(zoo, name)
    prompts = [prompt_tokens(V, n, 100 + i) for i, n in enumerate(lengths)]
    # float32 on pages of 8; bfloat16 on pages of 16, the smallest the matrix-core attention kernels
    # take, so that they meet portions beside single tokens on pages that were another request's.
    # The pool is the schedule's peak: every page is in use at some time, and later requests get
    # pages that earlier ones gave back.
    page = 8 if dtype == "float32" else 16
    steps = mixed_schedule(rng, lengths)
    n_pool = peak_pages(steps, page)
    eng = engines(name, dtype, page_size=page, max_tokens=n_pool * page, max_requests=4)
    got = {i: [] for i in range(len(lengths))}
    used = set()
    for entries, ends in steps:
        batch = [StepEntry(f"m{rid}", prompts[rid][lo:hi], list(range(hi - lo))) for rid, lo, hi in entries]
        out = eng.step(batch).cpu()
        for g in eng.cache.groups:
            for tab in g.tables.values():
                used.update(p for p in tab if p >= 0)
        at = 0
        for rid, lo, hi in entries:
            got[rid].append(out[at:at + hi - lo])
            at += hi - lo
        for rid in ends:
            eng.release(f"m{rid}")
        eng.cache.check()
    total_pages_asked = sum((n + page - 1) // page for n in lengths)
    assert total_pages_asked > n_pool >= len(used), "the schedule must make requests share pages over time"
    assert eng.free_pages() == [n_pool] * len(eng.cache.groups)
    for rid, n in enumerate(lengths):
        check_logits(torch.cat(got[rid]), zoo[1][name](prompts[rid]), dtype, f"{name} mixed request {rid}")


@pytest.mark.parametrize("name,dtype", [c for c in CASES if c[0] in ("A", "B", "C_keen", "C_sharp")])
def test_long_decoding(zoo, engines, name, dtype):
    eng = engines(name, dtype)
    toks = prompt_tokens(vocab_of(zoo, name), 330, 7)
    got = step_all(eng, "l", toks, [4] + [1] * 326)
    eng.release("l")
    check_logits(got, zoo[1][name](toks), dtype, f"{name} long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens(zoo, engines, name, dtype):
    eng = engines(name, dtype)
    for n in (1, 2, 3, 4):
        toks = prompt_tokens(vocab_of(zoo, name), n, 20 + n)
        for cuts in ([n], [1]):
            got = step_all(eng, "f", toks, cuts)
            eng.release("f")
            check_logits(got, zoo[1][name](toks), dtype, f"{name} first {n} tokens cut {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_wanted_places_only(zoo, engines, dtype):
    """`want` picks rows; a step that wants nothing returns nothing but still fills the cache."""
    from imparo_amd.engine import StepEntry
    eng = engines("B", dtype)
    toks = prompt_tokens(vocab_of(zoo, "B"), 40, 5)
    ref = zoo[1]["B"](toks)
    assert eng.step([StepEntry("x", toks[:20], [])]) is None
    out = eng.step([StepEntry("x", toks[20:], [19, 0, 7]), StepEntry("y", toks[:9], [8])]).cpu()
    eng.release("x"), eng.release("y")
    check_logits(out, torch.stack([ref[39], ref[20], ref[27], ref[8]]), dtype, "wanted places")


def test_placement_is_invisible(zoo, engines):
    """Permuted page placement gives the same bits (float32 and bfloat16)."""
    for dtype in DTYPES:
        toks = prompt_tokens(vocab_of(zoo, "C_keen"), 100, 9)
        base = step_all(engines("C_keen", dtype), "q", toks, [13, 1, 1, 40])
        engines("C_keen", dtype).release("q")
        eng = make_engine(zoo[0]["C_keen"], dtype)
        eng.cache.scramble(5)
        got = step_all(eng, "q", toks, [13, 1, 1, 40])
        assert any(t != sorted(t) or t[0] != 0 for g in eng.cache.groups for t in g.tables.values())
        assert torch.equal(got, base)


def test_cutting_and_batching_leave_float32_bits_alone(zoo, engines):
    """In float32 every sum runs in an order fixed by the position, so the way
    of cutting changes nothing at all."""
    eng = engines("B", "float32")
    toks = prompt_tokens(vocab_of(zoo, "B"), 90, 12)
    a = step_all(eng, "a", toks, [90])
    eng.release("a")
    b = step_all(eng, "a", toks, [3, 1, 20, 2])
    eng.release("a")
    assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", DTYPES)
def test_captured_decode_steps_equal_launched_ones(zoo, dtype):
    """Decode steps replay a captured graph. Replays are interleaved with
    launched work (a prompt portion of another request, a request that joins,
    one that leaves, contexts that grow past a table bucket) and every replay
    is compared, bit for bit, with the engine that launches each kernel."""
    from imparo_amd.engine import StepEntry
    V = vocab_of(zoo, "C_keen")
    prompts = [prompt_tokens(V, n, 300 + i) for i, n in enumerate((40, 37, 90, 260))]
    runs = []
    for use_graphs in (True, False):
        eng = make_engine(zoo[0]["C_keen"], dtype, page_size=16, max_tokens=4096, use_graphs=use_graphs)
        out = []
        for i in range(3):
            eng.step([StepEntry(f"r{i}", prompts[i][:-30], [])])
        for s in range(30):                          # three rows decode, teacher-forced
            batch = [StepEntry(f"r{i}", [prompts[i][len(prompts[i]) - 30 + s]], [0]) for i in range(3)]
            if s == 20:
                batch = batch[:2]                    # r2 sits this step out...
            out.append(eng.step(batch).cpu().clone())
            if s == 20:
                out.append(eng.step([batch_r2(prompts, s)]).cpu().clone())   # ...and goes on alone
            if s % 7 == 3:                           # launched work between replays
                lo = (s // 7) * 60
                out.append(eng.step([StepEntry("late", prompts[3][lo:lo + 60], [59])]).cpu().clone())
        if use_graphs:
            assert any(g.graph is not None for g in eng._graphs.values())
            assert len(eng._graphs) >= 2
        runs.append(torch.cat(out))
    assert torch.equal(runs[0], runs[1])
    ref = zoo[1]["C_keen"](prompts[0])
    check_logits(runs[0][0:1], ref[len(prompts[0]) - 30:len(prompts[0]) - 29], dtype, "first decoded row")


def test_captured_steps_are_kept_up_to_a_limit(zoo, monkeypatch):
    """More batch shapes than the engine keeps captures for: the one unused for longest is dropped
    and captured again when it comes back; every step equals the launched one."""
    from imparo_amd.engine import StepEntry
    import imparo_amd.engine.engine as engine_module
    monkeypatch.setattr(engine_module, "MAX_GRAPHS", 2)
    V = vocab_of(zoo, "A")
    prompts = [prompt_tokens(V, 30 + i, 500 + i) for i in range(3)]
    runs = []
    for use_graphs in (True, False):
        eng = make_engine(zoo[0]["A"], "bfloat16", page_size=16, max_tokens=1024, use_graphs=use_graphs)
        out = []
        for i in range(3):
            eng.step([StepEntry(f"r{i}", prompts[i][:10], [])])
        for s in range(10, 30):
            rows = (3, 2, 1, 3, 1)[s % 5]            # three shapes in turn with room for two
            out.append(eng.step([StepEntry(f"r{i}", [prompts[i][s]], [0]) for i in range(rows)]).cpu().clone())
            for i in range(rows, 3):                 # the others keep pace in a step of their own
                eng.step([StepEntry(f"r{i}", [prompts[i][s]], [])])
        if use_graphs:
            assert len(eng._graphs) == 2
        runs.append(torch.cat(out))
    assert torch.equal(runs[0], runs[1])


def batch_r2(prompts, s):
    from imparo_amd.engine import StepEntry
    return StepEntry("r2", [prompts[2][len(prompts[2]) - 30 + s]], [0])


def test_a_step_that_does_not_fit_changes_nothing(zoo):
    from imparo_amd.engine import StepEntry
    from imparo_amd.cache import OutOfPages
    eng = make_engine(zoo[0]["A"], "float32", page_size=8, max_tokens=64, max_requests=2)
    toks = prompt_tokens(vocab_of(zoo, "A"), 60, 3)
    ref = zoo[1]["A"](toks)
    first = eng.step([StepEntry("a", toks[:30], list(range(30)))]).cpu()
    free = eng.free_pages()
    with pytest.raises(OutOfPages):      # a's 10 more fit, b's 40 do not: neither advances
        eng.step([StepEntry("a", toks[30:40], [0]), StepEntry("b", toks[:40], [0])])
    assert eng.free_pages() == free and eng.length("a") == 30 and not eng.is_live("b")
    rest = eng.step([StepEntry("a", toks[30:], list(range(30)))]).cpu()
    check_logits(torch.cat([first, rest]), ref, "float32", "after a refused step")
    with pytest.raises(OutOfPages):      # the pool holds 64 positions
        eng.step([StepEntry("a", toks[:10], [])])
    eng.release("a")
    assert eng.free_pages() == [8]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tokens_fed_from_the_device(zoo, dtype):
    """A request's single token may be named as an element of an int32 vector on the device
    (where the sampling kernel left it): the step gives the logits it gives for the id itself,
    launch by launch, captured, and beside a portion of a prompt."""
    from imparo_amd.engine import StepEntry, DeviceToken, StepError
    vocab = vocab_of(zoo, "B")
    prompts = [prompt_tokens(vocab, n, 30 + n) for n in (12, 7, 20)]
    nxt = [prompt_tokens(vocab, 6, 90 + i) for i in range(3)]
    runs = []
    for from_device in (False, True):
        eng = make_engine(zoo[0]["B"], dtype, page_size=8, max_tokens=256, max_requests=4)
        for i in (0, 1):
            eng.step([StepEntry(i, prompts[i], [])])
        out = []
        for s in range(6):                     # steps 0..: eager, capture, replays; step 4 brings a prompt along
            ids = [nxt[0][s], nxt[1][s]]
            src = torch.tensor([7, ids[1], 3, ids[0]], dtype=torch.int32, device=eng.device)
            toks = [[DeviceToken(src, 3)], [DeviceToken(src, 1)]] if from_device else [[ids[0]], [ids[1]]]
            entries = [StepEntry(0, toks[0], [0]), StepEntry(1, toks[1], [0])]
            if s == 4:
                entries.insert(1, StepEntry(2, prompts[2], [19]))
            out.append(eng.step(entries).clone())     # the logits tensor is the engine's: the next step writes there
        runs.append(torch.cat(out).cpu())
        if from_device:
            with pytest.raises(StepError, match="device token"):
                eng.step([StepEntry(0, [DeviceToken(src, 4)], [0])])
            with pytest.raises(StepError, match="device token"):
                eng.step([StepEntry(0, [DeviceToken(src.long(), 0)], [0])])
            with pytest.raises(StepError, match="device token"):
                eng.step([StepEntry(0, [DeviceToken(src, 0)], [0]), StepEntry(1, [DeviceToken(src.clone(), 0)], [0])])
            assert eng.length(0) == 12 + 6
    assert torch.equal(runs[0], runs[1])
    ref = zoo[1]["B"](prompts[0] + nxt[0])
    check_logits(runs[0][0:1], ref[12:13], dtype, "first decoded row")


def test_pool_sizing_and_the_bound_on_a_steps_tokens(zoo):
    from imparo_amd.engine import Engine, StepEntry, StepError
    vocab = vocab_of(zoo, "C")
    # model C has two cache groups (all keys; a window): one number for both, or one each
    eng = Engine(zoo[0]["C"], dtype="bfloat16", page_size=16, num_pages=[9, 4], max_requests=2, max_step_tokens=40)
    assert [g.pool.n_pages for g in eng.cache.groups] == [9, 4]
    toks = prompt_tokens(vocab, 60, 3)
    with pytest.raises(StepError, match="max_step_tokens"):
        eng.step([StepEntry("a", toks[:41], [])])
    with pytest.raises(StepError, match="max_step_tokens"):
        eng.step([StepEntry("a", toks[:30], []), StepEntry("b", toks[:11], [])])
    assert not eng.is_live("a") and eng.free_pages() == [9, 4]
    got = torch.cat([eng.step([StepEntry("a", toks[:40], list(range(40)))]).cpu(),
                     eng.step([StepEntry("a", toks[40:], list(range(20)))]).cpu()])
    check_logits(got, zoo[1]["C"](toks), "bfloat16", "two cache groups with pools of their own")
    # a budget in bytes: pages of 16 positions x (5 kv heads x 16 x 2 arrays x 2 bytes) x 3 attention sites
    per_page = 16 * (5 * 16 * 2 * 2) * 3
    eng = Engine(zoo[0]["C"], dtype="bfloat16", page_size=16, kv_budget_bytes=12 * per_page + 100, max_requests=2)
    assert [g.pool.n_pages for g in eng.cache.groups] == [12, 12]
    assert sum(t.numel() * t.element_size() for a in eng.storage.paged.values() for t in a.values()) == 12 * per_page
    with pytest.raises(ValueError, match="one of"):
        Engine(zoo[0]["C"], max_tokens=64, num_pages=3)


def test_refused_batches(zoo, engines):
    from imparo_amd.engine import StepEntry, StepError
    eng = engines("A", "float32")
    with pytest.raises(StepError, match="outside the vocabulary"):
        eng.step([StepEntry("r", [1, 256], [0])])
    with pytest.raises(StepError, match="twice"):
        eng.step([StepEntry("r", [1], [0]), StepEntry("r", [2], [0])])
    with pytest.raises(StepError, match="wanted place"):
        eng.step([StepEntry("r", [1, 2], [2])])
    with pytest.raises(StepError, match="no tokens"):
        eng.step([StepEntry("r", [], [])])
    assert not eng.is_live("r")


def test_run_order_with_a_layer_twice_and_a_borrowed_cache(zoo, tmp_path):
    """The order layers run in is data: a plan that runs layer 1 twice, the
    second time reading the first call's keys and values, and layer 0 twice
    with a state of its own each time."""
    import dataclasses, json, shutil
    from imparo_amd.config import register_architecture, Lfm2Config, LayerCall
    from imparo_amd.config import lfm2
    order = [(0, None), (1, None), (1, 1), (2, None), (0, None), (3, None)]

    def build(cfg):
        plan = lfm2.build_plan(cfg)
        return dataclasses.replace(plan, architecture="TestLfm2Reordered",
                                   order=[LayerCall(l, c) for l, c in order])
    register_architecture("TestLfm2Reordered", Lfm2Config.from_dict, build)
    d = str(tmp_path / "reordered")
    shutil.copytree(zoo[0]["A_sharp"], d)
    cfg = json.load(open(os.path.join(d, "config.json")))
    cfg["architectures"] = ["TestLfm2Reordered"]
    json.dump(cfg, open(os.path.join(d, "config.json"), "w"))
    toks = prompt_tokens(256, 80, 31)
    ref = zoo[1]["A_sharp"](toks, order)
    assert not torch.allclose(ref, zoo[1]["A_sharp"](toks), atol=1e-3)
    eng = make_engine(d, "float32")
    assert len(eng.cache.fixed_sites) == 3 and len(eng.cache.groups[0].sites) == 2
    check_logits(step_all(eng, "o", toks, [9, 1, 1, 30, 2]), ref, "float32", "reordered float32")
    # the same order on the keen weights in bfloat16
    d2 = str(tmp_path / "reordered_keen")
    shutil.copytree(zoo[0]["A_keen"], d2)
    json.dump(cfg, open(os.path.join(d2, "config.json"), "w"))
    check_logits(step_all(make_engine(d2, "bfloat16"), "o", toks, [9, 1, 1, 30, 2]), zoo[1]["A_keen"](toks, order),
                 "bfloat16", "reordered bfloat16")
