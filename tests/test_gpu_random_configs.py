"""Configurations drawn at random (fixed seeds): every size and option the architecture's config.json
carries varies at once -- head size in steps of 16 up to 256, heads and groups, the number of layers
and their kinds (all conv, all attention, windows), vocabulary, feed-forward size given or adjusted,
conv taps and bias, tied or separate head, eps, rope base -- and each model is stepped through a
random mixed schedule (up to four live requests, portions beside single tokens, a pool at the
schedule's peak so that pages are used again) against the plain implementation, in both dtypes."""
import random

import pytest
import torch

from gpu_helpers import make_engine, mixed_schedule, peak_pages
from tolerances import check_logits

pytestmark = pytest.mark.gpu


def random_config(rng):
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
    heads = rng.choice([h for h in (1, 2, 3, 4, 5, 6, 8, 12) if h * head_dim <= 768])
    kv_heads = rng.choice([d for d in range(1, heads + 1) if heads % d == 0])
    n_layers = rng.randint(1, 5)
    kinds = [rng.choice(["conv", "conv", "full_attention", "sliding_attention"]) for _ in range(n_layers)]
    config = dict(architectures=["Lfm2ForCausalLM"], model_type="lfm2", max_position_embeddings=1024,
                  vocab_size=rng.randint(40, 900), hidden_size=heads * head_dim, num_hidden_layers=n_layers,
                  layer_types=kinds, num_attention_heads=heads, num_key_value_heads=kv_heads,
                  conv_L_cache=rng.randint(2, 8), conv_bias=rng.random() < 0.5, tie_embedding=rng.random() < 0.5,
                  rope_theta=rng.choice([1e4, 5e5, 1e6]), norm_eps=rng.choice([1e-5, 1e-6, 1e-3]))
    if rng.random() < 0.5:
        config.update(block_auto_adjust_ff_dim=True, block_ff_dim=rng.randint(60, 700),
                      block_multiple_of=rng.choice([8, 16, 40, 64]), block_ffn_dim_multiplier=rng.choice([1.0, 0.7, 1.3]))
    else:
        config.update(block_auto_adjust_ff_dim=False, block_ff_dim=rng.choice([rng.randint(24, 400), 8 * rng.randint(3, 50)]))
    if "sliding_attention" in kinds:
        config["sliding_window"] = rng.randint(5, 150)
    return config


@pytest.mark.parametrize("draw", range(12))
def test_a_random_configuration_in_a_mixed_schedule(draw, tmp_path):
    from imparo_amd import write_random_model
    from imparo_amd.engine import StepEntry
    from plain_lfm2 import PlainLfm2
    rng = random.Random(7919 * draw + 11)
    config = random_config(rng)
    folder = str(tmp_path / "model")
    write_random_model(config, 100 + draw, folder)
    plain = PlainLfm2(folder)
    vocab = config["vocab_size"]
    for dtype in ("float32", "bfloat16"):
        page = rng.choice([8, 16, 32, 64])
        lengths = [rng.choice([1, 2, 9, 33, 64, 65, 70, 121, 129, 250]) for _ in range(rng.randint(3, 6))]
        g = torch.Generator().manual_seed(draw)
        prompts = [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]
        steps = mixed_schedule(rng, lengths, sizes=(1, 1, 1, 1, 2, 2, 3, 5, 9, 16, 40, 63, 64, 65, 130))
        engine = make_engine(folder, dtype, max_tokens=peak_pages(steps, page) * page, page_size=page, max_requests=4)
        got = {rid: [] for rid in range(len(lengths))}
        for entries, ends in steps:
            # some entries want only some of their places, some none
            wants = [sorted(rng.sample(range(hi - lo), rng.randint(0, hi - lo))) if rng.random() < 0.3
                     else list(range(hi - lo)) for _, lo, hi in entries]
            out = engine.step([StepEntry(f"r{rid}", prompts[rid][lo:hi], w) for (rid, lo, hi), w in zip(entries, wants)])
            at = 0
            for (rid, lo, hi), w in zip(entries, wants):
                for j in w:
                    got[rid].append((lo + j, out[at].cpu()))
                    at += 1
            for rid in ends:
                engine.release(f"r{rid}")
            engine.cache.check()
        for rid, rows in got.items():
            if rows:
                ref = plain.logits(prompts[rid])
                check_logits(torch.stack([r for _, r in rows]), ref[[p for p, _ in rows]], dtype,
                             f"draw {draw} ({config}) {dtype} page {page} request {rid}")
