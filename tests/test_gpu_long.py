"""Long contexts and a serving workload. Up to some 4,000 tokens both dtypes
are held to the plain implementation; where it cannot follow (16,500 tokens)
the bfloat16 matrix-core path is held to the engine's own float32 path, and
continuous batching under page pressure is held to each request run alone."""
import random

import pytest
import torch

from conftest import assert_varied, prompt_tokens
from gpu_helpers import assert_picks_near_best, make_engine
from tolerances import BF16_REL, check_logits

pytestmark = pytest.mark.gpu

LONG = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=512, hidden_size=256,
    num_hidden_layers=4, layer_types=["conv", "full_attention", "sliding_attention", "full_attention"],
    num_attention_heads=4, num_key_value_heads=2, block_auto_adjust_ff_dim=False, block_ff_dim=512,
    conv_L_cache=3, conv_bias=False, rope_theta=1000000.0, tie_embedding=True, norm_eps=1e-5,
    max_position_embeddings=32768, sliding_window=700,
)


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    from imparo_amd import write_random_model
    d = str(tmp_path_factory.mktemp("long"))
    write_random_model(LONG, 5, d)
    return d


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_thousand_tokens_against_the_plain_implementation(long_model, dtype):
    """4,230 tokens: two portions of 2,048 (32 query tiles over up to 64 key tiles, the window of
    700 giving pages back on the way), a short portion, then single tokens through captured steps
    whose keys are walked in 17 splits. Every row of logits is compared."""
    from plain_lfm2 import PlainLfm2
    from imparo_amd.engine import StepEntry
    N = 4196
    toks = prompt_tokens(512, N + 34, 77)
    eng = make_engine(long_model, dtype, page_size=64, max_tokens=N + 128, max_requests=2)
    out = []
    for lo, hi in ((0, 2048), (2048, 4096), (4096, N)):
        out.append(eng.step([StepEntry("l", toks[lo:hi], list(range(hi - lo)))]).cpu())
    for i in range(N, N + 34):
        out.append(eng.step([StepEntry("l", toks[i:i + 1], [0])]).cpu().clone())
    ref = PlainLfm2(long_model).logits(toks)
    assert len(set(ref.argmax(-1).tolist())) >= 20        # the model's answers move with the context
    check_logits(torch.cat(out), ref, dtype, f"4,230 tokens {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_borrowed_cache_at_head_size_64(long_model, tmp_path, dtype):
    """A run order in which attention layer 1 runs twice, the second time on the first call's keys and
    values, decoded token by token. In bfloat16 with heads of 64 the call that owns the cache writes the
    new key inside its attention launch; the call that borrows must find it there and may not weigh in
    a key of its own."""
    import dataclasses, json, os, shutil
    from plain_lfm2 import PlainLfm2
    from imparo_amd.config import register_architecture, Lfm2Config, LayerCall, lfm2
    from gpu_helpers import step_all
    order = [(0, None), (1, None), (1, 1), (2, None), (3, None)]

    def build(cfg):
        plan = lfm2.build_plan(cfg)
        return dataclasses.replace(plan, architecture="TestLfm2Borrowing", order=[LayerCall(l, c) for l, c in order])
    register_architecture("TestLfm2Borrowing", Lfm2Config.from_dict, build)
    d = str(tmp_path / "borrowing")
    shutil.copytree(long_model, d)
    cfg = json.load(open(os.path.join(d, "config.json")))
    cfg["architectures"] = ["TestLfm2Borrowing"]
    json.dump(cfg, open(os.path.join(d, "config.json"), "w"))
    toks = prompt_tokens(512, 130, 12)
    plain = PlainLfm2(long_model)
    ref = plain.logits(toks, order)
    assert not torch.allclose(ref, plain.logits(toks), atol=1e-3)        # the second call matters
    eng = make_engine(d, dtype, page_size=64, max_tokens=512, max_requests=2)
    got = step_all(eng, "b", toks, [61] + [1] * 40 + [9] + [1] * 20)
    check_logits(got, ref, dtype, f"borrowed cache {dtype}")


def test_long_context_against_the_plain_implementation(long_model):
    """16,500 tokens in portions of 2,048 (tiles of 64 queries over hundreds of
    key tiles, a window of 700 that gives pages back), two short portions (their
    keys walked in parts), then single tokens over more than 64 splits of 256
    keys, through captured steps. Both dtypes are held to the plain implementation
    at every row that was asked for, under the bound for this many keys, and the
    bfloat16 run to the float32 run."""
    from plain_lfm2 import PlainLfm2
    from imparo_amd.engine import StepEntry
    from tolerances import bound
    N = 16500
    toks = prompt_tokens(512, N + 137 + 40, 99)
    asked = [r for lo in range(0, N, 2048) for r in range(min(N, lo + 2048) - 8, min(N, lo + 2048))]
    asked += list(range(N, N + 137 + 40))
    ref = PlainLfm2(long_model).logits(toks)[asked]
    runs = {}
    for dtype in ("float32", "bfloat16"):
        eng = make_engine(long_model, dtype, page_size=64, max_tokens=N + 256, max_requests=2)
        out = []
        for lo in range(0, N, 2048):
            hi = min(N, lo + 2048)
            out.append(eng.step([StepEntry("l", toks[lo:hi], list(range(hi - lo - 8, hi - lo)))]).cpu())
        for lo, hi in ((N, N + 100), (N + 100, N + 137)):
            out.append(eng.step([StepEntry("l", toks[lo:hi], list(range(hi - lo)))]).cpu())
        for i in range(N + 137, N + 137 + 40):
            out.append(eng.step([StepEntry("l", toks[i:i + 1], [0])]).cpu().clone())
        held = eng.cache.held_pages("l")
        assert held[0] == (N + 177 + 63) // 64 and held[1] <= 700 // 64 + 3    # the window's group holds a dozen pages
        runs[dtype] = torch.cat(out)
        check_logits(runs[dtype], ref, dtype, f"16,677 tokens, {dtype}", rel=bound(dtype, len(LONG["layer_types"]), N + 177))
    check_logits(runs["bfloat16"], runs["float32"], "bfloat16", "long context")


@pytest.fixture(scope="module")
def loud_long_model(tmp_path_factory):
    """The same shape with louder layers: a request's continuation then moves
    with every token, so an output that survived pre-emption, waiting and
    batching was recomputed from the right tokens and the right state."""
    from imparo_amd import write_random_model
    d = str(tmp_path_factory.mktemp("loud_long"))
    write_random_model(LONG, 5, d, layer_gain=8.0)
    return d


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_serving_workload_under_page_pressure(loud_long_model, dtype):
    """32 requests in waves, prompts of 20..600 tokens, 5..40 new tokens each, a pool that holds
    about a third of them at once: every output equals the request's output when it runs alone.
    In bfloat16 a request that runs alone takes other kernels than it took in a batch (the fused
    launches of steps with few rows), so a near-tie may fall the other way; there every token a
    request was given must be among the plain implementation's best for the tokens before it,
    to twice the bound on a logit (two logits, each off by the bound, can swap places)."""
    long_model = loud_long_model
    from imparo_amd.engine import Engine
    from imparo_amd.engine.scheduler import Scheduler, generate
    from imparo_amd.sampling import Sampler, SamplingParams
    rng = random.Random(3)
    reqs = [(prompt_tokens(512, rng.randint(20, 600), 500 + i), rng.randint(5, 40)) for i in range(32)]
    eng = Engine(long_model, dtype=dtype, page_size=16, max_tokens=3200, max_requests=12)
    sched = Scheduler(eng, Sampler(eng.device).pick, max_batch_tokens=512, max_running=12, portion=128)
    pending = list(enumerate(reqs))
    while pending or sched.has_work():
        if pending and (not sched.has_work() or rng.random() < 0.3):
            for _ in range(min(8, len(pending))):                 # a wave arrives
                i, (prompt, n) = pending.pop(0)
                sched.add(i, prompt, SamplingParams(max_tokens=n))
        if sched.has_work():
            sched.step()
            eng.cache.check()
    assert any(e[0] == "preempt" for e in sched.log) and any(e[0] == "wait" for e in sched.log)
    assert eng.free_pages() == [200, 200] and eng.cache.slots.n_free == 12
    checked = rng.sample(range(32), 10)
    assert_varied([sched.finished[i].generated for i in checked if reqs[i][1] >= 8])
    if dtype == "float32":
        alone = Engine(long_model, dtype="float32", page_size=16, max_tokens=1024, max_requests=2)
        for i in checked:
            prompt, n = reqs[i]
            assert sched.finished[i].finish_reason == "length"
            assert sched.finished[i].generated == generate(alone, [prompt], max_tokens=n)[0], f"request {i}"
        return
    from plain_lfm2 import PlainLfm2
    plain = PlainLfm2(long_model)
    for i in checked:
        prompt, n = reqs[i]
        assert sched.finished[i].finish_reason == "length" and len(sched.finished[i].generated) == n
        assert_picks_near_best(plain, prompt, sched.finished[i].generated, 2 * BF16_REL, f"request {i}")
