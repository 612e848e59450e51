"""The native step program against the parts run one by one: both issue the same kernels with the
same arguments (with the program's folding of norms switched off), so every step's logits are the same
bits, in both dtypes, launch by launch and through captured graphs. Then the folded norms against the
plain implementation, the engine's first steps when nothing has run before them, and `Engine.warm`."""
import random

import pytest
import torch

from conftest import prompt_tokens
from gpu_helpers import make_engine, mixed_schedule, peak_pages
from tolerances import check_logits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_one_native_call_and_parts_one_by_one_give_the_same_bits(model_dirs, name, dtype, graphs):
    from imparo_amd.engine import StepEntry
    from tiny_configs import CONFIGS
    vocab = CONFIGS[name][0]["vocab_size"]
    lengths = [70, 33, 120, 18, 64, 91]
    prompts = [prompt_tokens(vocab, n, 40 + i) for i, n in enumerate(lengths)]
    steps = mixed_schedule(random.Random(7), lengths, sizes=(1, 1, 1, 1, 2, 3, 9, 16, 40))
    pool = peak_pages(steps, 16)
    engines = [make_engine(model_dirs[name], dtype, page_size=16, max_tokens=pool * 16, max_requests=4,
                           use_graphs=graphs, native_step=native, fold_norms=False) for native in (True, False)]
    assert engines[0].program is not None and engines[1].program is None
    for entries, ends in steps:
        outs = [eng.step([StepEntry(f"r{rid}", prompts[rid][lo:hi], list(range(hi - lo))) for rid, lo, hi in entries])
                for eng in engines]
        assert torch.equal(outs[0], outs[1]), f"{name} {dtype}: the two ways differ at a step of {entries}"
        for rid in ends:
            for eng in engines:
                eng.release(f"r{rid}")
    for eng in engines:
        assert eng.free_pages() == [pool] * len(eng.free_pages())
    assert not graphs or engines[0]._graphs, "single-token steps of this schedule go through captured graphs"


@pytest.mark.parametrize("native", [True, False])
def test_wanting_nothing_and_wanting_some_rows(model_dirs, plain_models, native):
    from imparo_amd.engine import StepEntry
    toks = prompt_tokens(256, 40, 3)
    eng = make_engine(model_dirs["A"], "float32", native_step=native)
    assert eng.step([StepEntry("a", toks[:30], [])]) is None
    out = eng.step([StepEntry("a", toks[30:], [0, 9])]).cpu()
    check_logits(out, plain_models["A"].logits(toks)[[30, 39]], "float32", "two wanted rows")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_steps_are_single_tokens_through_captured_graphs(dtype, tmp_path_factory):
    """Every prompt has one token, so nothing but single-token steps ever runs: the engine's first
    step of 8 rows is captured at once (no step ran launch by launch before it), and so is the
    first step of 20 rows, which takes kernels of other files (the head norm and rotation on its
    own, the unfused conv, the 17-to-64-row products). Heads of 64 so that the fused launch is taken
    at 8 rows. The code of every file of kernels is on the device when the engine is built."""
    from imparo_amd import write_random_model
    from imparo_amd.engine import StepEntry
    from plain_lfm2 import PlainLfm2
    cfg = dict(architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=300, hidden_size=256,
               num_hidden_layers=3, layer_types=["conv", "full_attention", "conv"], num_attention_heads=4,
               num_key_value_heads=2, block_auto_adjust_ff_dim=False, block_ff_dim=384, conv_L_cache=3, conv_bias=False,
               rope_theta=10000.0, tie_embedding=True, norm_eps=1e-5, max_position_embeddings=512)
    d = str(tmp_path_factory.mktemp("heads64"))
    write_random_model(cfg, 9, d)
    plain = PlainLfm2(d)
    seqs = [prompt_tokens(300, 6, 200 + i) for i in range(20)]
    refs = [plain.logits(s) for s in seqs]
    eng = make_engine(d, dtype, page_size=64, max_tokens=20 * 64, max_requests=20)
    for j in range(3):
        out = eng.step([StepEntry(i, [seqs[i][j]], [0]) for i in range(8)]).cpu()
        check_logits(out, torch.stack([refs[i][j] for i in range(8)]), dtype, f"8 rows, token {j}")
    assert list(eng._graphs) == [(8, 8)]
    for j in range(3):
        rows = [(i, j + 3 if i < 8 else j) for i in range(20)]
        out = eng.step([StepEntry(i, [seqs[i][t]], [0]) for i, t in rows]).cpu()
        check_logits(out, torch.stack([refs[i][t] for i, t in rows]), dtype, f"20 rows, step {j}")
    assert sorted(eng._graphs) == [(8, 8), (20, 8)]


def test_warm_captures_shapes_before_they_are_met(model_dirs, plain_models):
    from imparo_amd.engine import StepEntry
    eng = make_engine(model_dirs["B"], "bfloat16", page_size=16, max_tokens=1024, max_requests=4)
    assert eng.warm(rows=[1, 2, 3], contexts=[100, 300]) == 6
    shapes = set(eng._graphs)
    assert eng.warm(rows=[2], contexts=[100]) == 0
    seqs = [prompt_tokens(384, 90 + 9 * i, 20 + i) for i in range(3)]
    refs = [plain_models["B"].logits(s) for s in seqs]
    for i, s in enumerate(seqs):
        eng.step([StepEntry(i, s[:-4], [])])
    for j in range(4):
        out = eng.step([StepEntry(i, [s[len(s) - 4 + j]], [0]) for i, s in enumerate(seqs)]).cpu()
        check_logits(out, torch.stack([r[len(s) - 4 + j] for r, s in zip(refs, seqs)]), "bfloat16", f"warmed step {j}")
    assert set(eng._graphs) == shapes, "the steps ran from graphs that warm() had captured"
    # more shapes than the engine keeps by default: all of what was asked for stays
    eng.max_graphs = 4
    assert eng.warm(rows=[1, 2, 3, 4], contexts=[100, 300, 900]) == 6 and len(eng._graphs) == 12


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_norms_folded_into_the_products_around_them(model_dirs, plain_models, name):
    """Steps of at most 16 single tokens with every norm between two products folded away: the
    product before it adds to the stream and leaves sums of squares and weighted rows, the product
    behind it scales at its end. Five requests decode ten tokens each after prompts of different
    lengths; every row is held to the plain implementation, and the folded engine to the unfolded
    one within the same bound."""
    from imparo_amd.engine import StepEntry
    from tiny_configs import CONFIGS
    vocab = CONFIGS[name][0]["vocab_size"]
    seqs = [prompt_tokens(vocab, n + 10, 60 + i) for i, n in enumerate((1, 7, 16, 33, 50))]
    refs = [plain_models[name].logits(s) for s in seqs]
    outs = {}
    for fold in (True, False):
        eng = make_engine(model_dirs[name], "bfloat16", page_size=16, max_tokens=512, max_requests=8, fold_norms=fold)
        shape = eng._args
        for i, s in enumerate(seqs):
            eng.step([StepEntry(i, s[:-10], [])])
        got = []
        for j in range(10):
            out = eng.step([StepEntry(i, [s[len(s) - 10 + j]], [0]) for i, s in enumerate(seqs)]).cpu()
            got.append(out.clone())
            check_logits(out, torch.stack([r[len(s) - 10 + j] for r, s in zip(refs, seqs)]), "bfloat16",
                         f"{name}, norms folded: {fold}, step {j}")
        outs[fold] = torch.stack(got)
        used = eng.program.needs(eng._step_args_for_rows(5))
        assert ("fold_ssq" in used) == fold, "the decode step of five rows folds its norms exactly when asked to"
    assert not torch.equal(outs[True], outs[False])     # two ways of rounding
