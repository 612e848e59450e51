"""Generation through the entry points: greedy against the plain
implementation, temperature sampling with a fixed seed in portions mixed with
decodes, pre-emption by recompute, the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import assert_varied, prompt_tokens, ROOT
from gpu_helpers import assert_picks_near_best
from tolerances import BF16_REL

pytestmark = pytest.mark.gpu


def plain_sample(plain, prompt, n, temperature, seed):
    from imparo_amd.sampling import uniform_for
    seq, out = list(prompt), []
    for i in range(n):
        row = plain.logits(seq)[-1].double()
        if temperature <= 0:
            tok = int(torch.argmax(row))
        else:
            cdf = torch.cumsum(torch.softmax(row / temperature, 0), 0)
            tok = int(torch.searchsorted(cdf, torch.tensor(uniform_for(seed, i), dtype=torch.float64), right=True))
            tok = min(tok, row.shape[0] - 1)
        out.append(tok)
        seq.append(tok)
    return out


def test_greedy_generation_tiny_a(model_dirs, plain_models):
    """Tiny A's workload: prompts of 5, 17 and 31 tokens, 16 greedy tokens each."""
    from imparo_amd import generate
    prompts = [prompt_tokens(256, n, 40 + n) for n in (5, 17, 31)]
    want = [plain_models["A"].greedy(p, 16) for p in prompts]
    got = generate(model_dirs["A"], prompts, max_tokens=16, dtype="float32", page_size=8)
    assert got == want
    os.environ["IMPARO_BATCH"] = "4"          # 4-token portions
    try:
        got = generate(model_dirs["A"], prompts, max_tokens=16, dtype="float32", page_size=8, max_batch_tokens=9)
    finally:
        del os.environ["IMPARO_BATCH"]
    assert got == want


def test_greedy_generation_follows_every_token(loud_model_dirs, loud_plain_models):
    """The same workloads on models whose continuation moves with every token
    (with the stated spreads it is one token repeated): greedy, whole and in
    small portions under a small budget, Tiny B with its biases and its head."""
    from imparo_amd import generate
    for name, vocab, lens in (("A", 256, (5, 17, 31)), ("B", 384, (1, 9, 40, 63))):
        prompts = [prompt_tokens(vocab, n, 40 + n) for n in lens]
        want = [loud_plain_models[name].greedy(p, 16) for p in prompts]
        assert_varied(want)
        assert generate(loud_model_dirs[name], prompts, max_tokens=16, dtype="float32", page_size=8) == want
        os.environ["IMPARO_BATCH"] = "4"
        try:
            got = generate(loud_model_dirs[name], prompts, max_tokens=16, dtype="float32", page_size=8,
                           max_batch_tokens=9)
        finally:
            del os.environ["IMPARO_BATCH"]
        assert got == want


def test_greedy_generation_bfloat16_stays_on_a_best_token(model_dirs, plain_models):
    """In bfloat16 a near-tie may fall the other way; every token the engine
    picks must be the plain implementation's best up to the logit tolerance."""
    from imparo_amd import generate
    prompts = [prompt_tokens(256, n, 40 + n) for n in (5, 17, 31)]
    got = generate(model_dirs["A"], prompts, max_tokens=16, dtype="bfloat16")
    for p, out in zip(prompts, got):
        assert len(out) == 16
        ref = plain_models["A"].logits(p + out)
        for i, tok in enumerate(out):
            row = ref[len(p) - 1 + i]
            assert row[tok] >= row.max() - 2 * BF16_REL * row.abs().max()


def test_temperature_sampling_tiny_b(model_dirs, plain_models):
    """Tiny B's workload: prompts of 1, 9, 40 and 63 tokens, 24 tokens each at
    temperature 0.8 under a fixed seed, in 7-token portions mixed with decodes."""
    from imparo_amd import generate
    prompts = [prompt_tokens(384, n, 60 + n) for n in (1, 9, 40, 63)]
    want = [plain_sample(plain_models["B"], p, 24, 0.8, 7 + i) for i, p in enumerate(prompts)]
    assert len({tuple(w) for w in want}) == 4 and want[0] != plain_models["B"].greedy(prompts[0], 24)
    os.environ["IMPARO_BATCH"] = "7"
    try:
        got = generate(model_dirs["B"], prompts, max_tokens=24, temperature=0.8, seed=7, dtype="float32",
                       page_size=8, max_batch_tokens=12)
        alone = [generate(model_dirs["B"], [p], max_tokens=24, temperature=0.8, seed=7 + i, dtype="float32")[0]
                 for i, p in enumerate(prompts[:2])]
    finally:
        del os.environ["IMPARO_BATCH"]
    assert got == want
    assert alone == want[:2]          # a request's draws do not depend on its batch


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("overlap", [False, True])
def test_preemption_by_recompute_keeps_greedy_outputs(loud_model_dirs, loud_plain_models, overlap, dtype):
    model_dirs, plain_models = loud_model_dirs, loud_plain_models
    from imparo_amd.engine import Engine
    from imparo_amd.engine.scheduler import Scheduler
    from imparo_amd.sampling import Sampler, SamplingParams
    prompts = [prompt_tokens(256, n, 80 + n) for n in (20, 22, 18)]
    want = [plain_models["A"].greedy(p, 20) for p in prompts]
    assert_varied(want)          # a recompute that dropped or repeated a token would change what follows
    eng = Engine(model_dirs["A"], dtype=dtype, page_size=8, max_tokens=10 * 8, max_requests=4)
    sampler = Sampler(eng.device)
    sched = Scheduler(eng, sampler.pick, max_batch_tokens=64, pick_async=sampler.pick_async if overlap else None)
    for i, p in enumerate(prompts):
        sched.add(i, p, SamplingParams(max_tokens=20))
    done = sched.run()
    assert any(e[0] == "preempt" for e in sched.log)
    assert eng.free_pages() == [10]
    if dtype == "float32":
        assert [done[i].generated for i in range(3)] == want
        return
    # bfloat16 may turn a near-tie the other way; each token must be among the best for its own prefix
    for i, p in enumerate(prompts):
        assert len(done[i].generated) == 20
        assert_picks_near_best(plain_models["A"], p, done[i].generated, 2 * BF16_REL, f"request {i}")


def test_stop_token_and_entry_point_defaults(loud_model_dirs, loud_plain_models):
    from imparo_amd import generate
    p = prompt_tokens(256, 12, 5)
    full = loud_plain_models["A"].greedy(p, 10)
    assert_varied([full])
    at = next(i for i in range(3, 10) if full[i] not in full[:i])       # a token that comes first at place 3 or later
    # the reply ends at the stop token, which is not handed out
    got = generate(loud_model_dirs["A"], [p], max_tokens=10, dtype="float32", stop_token_ids=[full[at]])
    assert got == [full[:at]]
    # no prompts, no replies; a prompt without tokens is refused by name
    assert generate(loud_model_dirs["A"], []) == []
    with pytest.raises(ValueError, match="at least one prompt token"):
        generate(loud_model_dirs["A"], [p, []], max_tokens=2, dtype="float32")


def test_waiting_after_every_step_generates_the_same(loud_model_dirs):
    model_dirs = loud_model_dirs
    """By default a step is queued before the tokens of the step before are read back (they
    are fed from the device); overlap=False waits after every step. Same tokens either way:
    greedy and sampled, with a stop token that is noticed a step late, in both dtypes."""
    from imparo_amd import generate
    prompts = [prompt_tokens(384, n, 60 + n) for n in (3, 9, 40, 21, 2)]
    for dtype in ("float32", "bfloat16"):
        for kw in (dict(), dict(temperature=0.8, seed=5)):
            free = generate(model_dirs["B"], prompts, max_tokens=20, dtype=dtype, page_size=8, parallel=3,
                            max_batch_tokens=16, overlap=False, **kw)
            assert generate(model_dirs["B"], prompts, max_tokens=20, dtype=dtype, page_size=8, parallel=3,
                            max_batch_tokens=16, **kw) == free
            stops = [free[0][3], free[2][7], free[3][-1]]
            a = generate(model_dirs["B"], prompts, max_tokens=20, dtype=dtype, page_size=8, parallel=3,
                         max_batch_tokens=16, stop_token_ids=stops, overlap=False, **kw)
            b = generate(model_dirs["B"], prompts, max_tokens=20, dtype=dtype, page_size=8, parallel=3,
                         max_batch_tokens=16, stop_token_ids=stops, **kw)
            assert a == b and len(a[0]) <= 3 and all(t not in stops for out in a for t in out)


def test_command_line(loud_model_dirs, loud_plain_models, tmp_path):
    model_dirs = loud_model_dirs
    p = prompt_tokens(256, 9, 3)
    want = loud_plain_models["A"].greedy(p, 6)
    assert_varied([want])
    env = dict(os.environ, PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, "-m", "imparo_amd", "generate", "-m", model_dirs["A"], "--dtype", "float32",
                        "--input-ids", ",".join(map(str, p)), "--max-tokens", "6", "-np", "2", "-c", "64"],
                       capture_output=True, text=True, env=env, timeout=240)
    assert r.returncode == 0, r.stderr
    assert json.loads(r.stdout.splitlines()[0])["output_ids"] == want
    # a stop id given on the command line ends the reply before it; a small pool (--num-pages) changes nothing
    stop = next(t for i, t in enumerate(want) if i >= 2 and t not in want[:i])
    r = subprocess.run([sys.executable, "-m", "imparo_amd", "generate", "-m", model_dirs["A"], "--dtype", "float32",
                        "--input-ids", " ".join(map(str, p)), "--max-tokens", "6", "--stop-token-ids", f"{stop},255",
                        "--page-size", "8", "--num-pages", "3"],
                       capture_output=True, text=True, env=env, timeout=240)
    assert r.returncode == 0, r.stderr
    assert json.loads(r.stdout.splitlines()[0])["output_ids"] == want[:want.index(stop)]
    r = subprocess.run([sys.executable, "-m", "imparo_amd", "forward", "--dtype", "float32", "--decode", "5",
                        "--split", "0,4", "--scramble-kv", "--page-size", "8", model_dirs["A"]] + list(map(str, p)),
                       capture_output=True, text=True, env=env, timeout=240)
    assert r.returncode == 0, r.stdout + r.stderr
    trails = [l.split()[1:] for l in r.stdout.splitlines() if l.strip().startswith("trail")]
    assert trails == [list(map(str, want[:5]))] * 2
    assert "scramble-kv: max |delta| to identity placement: 0.000e+00" in r.stdout
    r = subprocess.run([sys.executable, "-m", "imparo_amd", "forward", "--dtype", "float32", "--decode", "4",
                        "--cobatch", "3", model_dirs["A"]] + list(map(str, p)),
                       capture_output=True, text=True, env=env, timeout=240)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "max |logit delta| together vs alone = 0.000e+00" in r.stdout
