"""The benchmark's own model, whole: LFM2-1.2B's 16 layers at their full sizes, random weights of
seed 2, held against the plain implementation in float32 and in bfloat16, each request whole, with its
last 32 tokens one by one, in portions of changing size down to two tokens, and mixed with other
requests on a pool no larger than the schedule's peak. The reference gates its kernels on the whole
model's logits (/root/reference/README.md:98-117,
/root/reference/crates/imparo-model/src/bin/imparo-forward.rs:1122-1126); this is that gate here.
The bounds come from tolerances.bound(dtype, 16), a rule of depth stated before this test ran."""
import os
import random
import sys

import pytest
import torch

from conftest import prompt_tokens
from gpu_helpers import make_engine, mixed_schedule, peak_pages, step_all
from tolerances import bound, check_logits

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
N_TOKENS = 104


@pytest.fixture(scope="module")
def full(tmp_path_factory):
    sys.path.insert(0, ROOT)
    from bench import LFM2_1_2B
    from imparo_amd import write_random_model
    from plain_lfm2 import PlainLfm2
    d = str(tmp_path_factory.mktemp("full_depth"))
    write_random_model(LFM2_1_2B, 2, d)
    plain = PlainLfm2(d)
    lengths = [N_TOKENS, 70, 45, 90, 66]
    prompts = [prompt_tokens(65536, n, 900 + i) for i, n in enumerate(lengths)]
    refs = [plain.logits(p) for p in prompts]
    layers = len(LFM2_1_2B["layer_types"])
    del plain
    return d, prompts, refs, layers


def _mixed(eng, prompts, seed):
    """Runs all prompts under a schedule of up to four live requests; returns every request's logits."""
    from imparo_amd.engine import StepEntry
    rng = random.Random(seed)
    lengths = [len(p) for p in prompts]
    steps = mixed_schedule(rng, lengths, sizes=(1, 1, 1, 2, 2, 3, 7, 17, 40, 64))
    got = {i: [] for i in range(len(prompts))}
    kinds = set()
    for entries, ends in steps:
        sizes = [hi - lo for _, lo, hi in entries]
        kinds.add((any(n == 1 for n in sizes), any(n > 1 for n in sizes)))
        out = eng.step([StepEntry(f"m{rid}", prompts[rid][lo:hi], list(range(hi - lo))) for rid, lo, hi in entries]).cpu()
        at = 0
        for rid, lo, hi in entries:
            got[rid].append(out[at:at + hi - lo])
            at += hi - lo
        for rid in ends:
            eng.release(f"m{rid}")
        eng.cache.check()
    assert (True, True) in kinds, "the schedule must put single tokens beside portions"
    return {rid: torch.cat(parts) for rid, parts in got.items()}


def _pool_for(prompts, seed):
    steps = mixed_schedule(random.Random(seed), [len(p) for p in prompts], sizes=(1, 1, 1, 2, 2, 3, 7, 17, 40, 64))
    pool = peak_pages(steps, 64)
    assert sum((len(p) + 63) // 64 for p in prompts) > pool          # pages are used again
    return pool


def _four_ways(d, dtype, prompts):
    toks = prompts[0]
    pool = _pool_for(prompts, 11)
    eng = make_engine(d, dtype, page_size=64, max_tokens=pool * 64, max_requests=4)
    runs = {}
    runs["whole"] = step_all(eng, "w", toks, [len(toks)])
    eng.release("w")
    runs["last 32 one by one"] = step_all(eng, "s", toks, [len(toks) - 32] + [1] * 32)
    eng.release("s")
    runs["changing portions"] = step_all(eng, "p", toks, [2, 31, 3, 2, 17, 5, 2, 40, 2])
    eng.release("p")
    mixed = _mixed(eng, prompts, 11)
    assert eng.free_pages() == [pool]
    runs["mixed"] = mixed[0]
    return runs, mixed


def test_full_depth_float32_four_ways(full):
    d, prompts, refs, layers = full
    rel = bound("float32", layers)
    runs, mixed = _four_ways(d, "float32", prompts)
    for what, got in runs.items():
        check_logits(got, refs[0], "float32", f"16 layers, float32, {what}", rel=rel)
        # in float32 every sum's order is a function of the position only: the same bits however cut
        assert torch.equal(got, runs["whole"]), f"float32 {what} differs from the whole prompt's bits"
    for rid, got in mixed.items():
        check_logits(got, refs[rid], "float32", f"16 layers, float32, mixed request {rid}", rel=rel)


def test_full_depth_bfloat16_four_ways(full):
    d, prompts, refs, layers = full
    rel = bound("bfloat16", layers)
    runs, mixed = _four_ways(d, "bfloat16", prompts)
    for what, got in list(runs.items()) + [(f"mixed request {r}", g) for r, g in mixed.items() if r]:
        ref = refs[0] if what in runs else refs[int(what.split()[-1])]
        check_logits(got, ref, "bfloat16", f"16 layers, bfloat16, {what}", rel=rel)
        # what a user sees: the token the engine would pick is one of the plain implementation's best.
        # (Two logits each within the bound can swap only if they lie within twice the bound.)
        picked = got.argmax(dim=-1)
        best = ref.max(dim=-1).values
        at_picked = ref.gather(1, picked[:, None])[:, 0]
        assert bool((best - at_picked <= 2 * rel * ref.abs().max()).all()), f"{what}: a picked token is far from the best"
