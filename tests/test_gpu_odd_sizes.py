"""Configurations at the edges of what the kernels take, end to end against the plain
implementation: 13 heads of 16 without groups, a vocabulary and a feed-forward width that are no
multiple of 8, 5 and 8 conv taps, head sizes of 48, 80, 96, 128, 160 and 256 (the last two beyond the
matrix-core attention kernels), a window that is no multiple of a page. Each runs a random
schedule of mixed batches (portions of up to 200 tokens beside single tokens, pages used again,
only some places wanted), in float32 and in bfloat16."""
import random

import pytest
import torch

from conftest import prompt_tokens
from gpu_helpers import make_engine, mixed_schedule
from tolerances import check_logits

pytestmark = pytest.mark.gpu


def _cfg(**kw):
    base = dict(architectures=["Lfm2ForCausalLM"], model_type="lfm2", conv_bias=False, tie_embedding=True,
                block_auto_adjust_ff_dim=False, max_position_embeddings=4096, rope_theta=10000.0, norm_eps=1e-5)
    base.update(kw)
    return base


ODD = {
    "13_heads_of_16": _cfg(vocab_size=1001, hidden_size=208, num_hidden_layers=3,
                           layer_types=["conv", "full_attention", "full_attention"], num_attention_heads=13,
                           num_key_value_heads=13, block_ff_dim=100, conv_L_cache=5),
    "heads_of_80": _cfg(vocab_size=77, hidden_size=240, num_hidden_layers=2, layer_types=["full_attention", "conv"],
                        num_attention_heads=3, num_key_value_heads=1, block_ff_dim=72, conv_L_cache=8, conv_bias=True),
    "heads_of_256": _cfg(vocab_size=130, hidden_size=512, num_hidden_layers=2, layer_types=["full_attention", "conv"],
                         num_attention_heads=2, num_key_value_heads=2, block_ff_dim=64, conv_L_cache=3),
    "heads_of_128_in_groups": _cfg(vocab_size=300, hidden_size=512, num_hidden_layers=2,
                                   layer_types=["full_attention", "conv"], num_attention_heads=4,
                                   num_key_value_heads=2, block_ff_dim=96, conv_L_cache=3),
    "heads_of_96": _cfg(vocab_size=150, hidden_size=288, num_hidden_layers=2, layer_types=["conv", "full_attention"],
                        num_attention_heads=3, num_key_value_heads=3, block_ff_dim=80, conv_L_cache=3),
    "six_heads_of_48": _cfg(vocab_size=99, hidden_size=288, num_hidden_layers=2,
                            layer_types=["full_attention", "full_attention"], num_attention_heads=6,
                            num_key_value_heads=2, block_ff_dim=120, conv_L_cache=3),
    "heads_of_160_window_33": _cfg(vocab_size=130, hidden_size=320, num_hidden_layers=2,
                                   layer_types=["sliding_attention", "full_attention"], num_attention_heads=2,
                                   num_key_value_heads=1, block_ff_dim=64, conv_L_cache=3, sliding_window=33),
}


@pytest.fixture(scope="module")
def odd_models(tmp_path_factory):
    from imparo_amd import write_random_model
    from plain_lfm2 import PlainLfm2
    out = {}
    for i, (name, cfg) in enumerate(ODD.items()):
        d = str(tmp_path_factory.mktemp(f"odd_{i}"))
        write_random_model(cfg, 20 + i, d)
        out[name] = (d, PlainLfm2(d))
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ODD))
def test_odd_sizes_in_mixed_batches(odd_models, name, dtype):
    from imparo_amd.engine import StepEntry
    d, plain = odd_models[name]
    V = ODD[name]["vocab_size"]
    rng = random.Random(len(name))
    page = rng.choice([8, 16, 64])
    lengths = [rng.choice([1, 2, 9, 33, 64, 65, 129, 250]) for _ in range(5)] + [140]
    prompts = [prompt_tokens(V, n, 700 + i) for i, n in enumerate(lengths)]
    n_pages = sum(sorted((n + page - 1) // page for n in lengths)[-4:]) + 1
    eng = make_engine(d, dtype, page_size=page, max_tokens=n_pages * page, max_requests=4)
    got = {i: [] for i in range(len(lengths))}
    for entries, ends in mixed_schedule(rng, lengths, sizes=(1, 1, 1, 2, 3, 9, 40, 64, 65, 200)):
        wants = [sorted(rng.sample(range(hi - lo), rng.randint(0, hi - lo))) if rng.random() < 0.3
                 else list(range(hi - lo)) for _, lo, hi in entries]
        out = eng.step([StepEntry(f"m{rid}", prompts[rid][lo:hi], w) for (rid, lo, hi), w in zip(entries, wants)])
        at = 0
        for (rid, lo, hi), w in zip(entries, wants):
            for j in w:
                got[rid].append((lo + j, out[at].cpu()))
                at += 1
        for rid in ends:
            eng.release(f"m{rid}")
        eng.cache.check()
    assert eng.free_pages() == [n_pages] * len(eng.cache.groups)
    for rid in range(len(lengths)):
        if got[rid]:
            ref = plain.logits(prompts[rid])
            check_logits(torch.stack([r for _, r in got[rid]]), ref[[p for p, _ in got[rid]]], dtype,
                         f"{name} {dtype} request {rid}")
