"""Layers of the benchmark's own width (hidden 2048, 32 heads of 64 over 8 kv
heads, feed-forward 8192, vocabulary 65536) with few layers, so that the plain
implementation can follow on the CPU: the kernels' paths for these sizes (the
128x128 MFMA tiles, the wide few-row products, the float4 norm, matrix-core
attention at head size 64, pages of 64) are compared end to end. The widths of
the two smaller checkpoints (hidden 1536 / 24 heads / feed-forward 6912, hidden
1024 / 16 heads / feed-forward 4608) run the same tests: the products' plans
(tile, stages, slices of K) and the attention's grouping of heads differ per
width, and each is met here before any measurement meets it (the reference
keeps one contract test per geometry,
/root/reference/crates/imparo-cuda/tests/lfm2_contract.rs:316-335)."""
import random

import pytest
import torch

from conftest import prompt_tokens
from gpu_helpers import make_engine, mixed_schedule, peak_pages, step_all
from tolerances import check_logits

pytestmark = pytest.mark.gpu

WIDE = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=65536, hidden_size=2048,
    num_hidden_layers=3, layer_types=["conv", "full_attention", "conv"],
    num_attention_heads=32, num_key_value_heads=8,
    block_auto_adjust_ff_dim=True, block_ff_dim=12288, block_multiple_of=256, block_ffn_dim_multiplier=1.0,
    conv_L_cache=3, conv_bias=False, rope_theta=1000000.0, tie_embedding=True, norm_eps=1e-5,
    max_position_embeddings=128000,
)


# (hidden, heads, block_ff_dim): the three LFM2 checkpoints' widths, three layers of each
WIDTHS = {"1.2B": (2048, 32, 12288), "700M": (1536, 24, 10240), "350M": (1024, 16, 6656)}


def _wide_model(tmp_path_factory, name):
    from imparo_amd import write_random_model
    from plain_lfm2 import PlainLfm2
    hidden, heads, ff = WIDTHS[name]
    cfg = dict(WIDE, hidden_size=hidden, num_attention_heads=heads, block_ff_dim=ff)
    d = str(tmp_path_factory.mktemp("wide_" + name.replace(".", "_")))
    write_random_model(cfg, 2, d)
    plain = PlainLfm2(d)
    assert plain.w["model.layers.0.feed_forward.w1.weight"].shape[0] == {"1.2B": 8192, "700M": 6912, "350M": 4608}[name]
    toks = prompt_tokens(65536, 200, 77)
    return d, toks, plain.logits(toks), plain


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    return _wide_model(tmp_path_factory, "1.2B")


@pytest.fixture(scope="module", params=["700M", "350M"])
def narrower(request, tmp_path_factory):
    return _wide_model(tmp_path_factory, request.param)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_width_layers(wide, dtype):
    _whole_and_portions(wide, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_smaller_checkpoints_widths(narrower, dtype):
    _whole_and_portions(narrower, dtype)


def _whole_and_portions(model, dtype):
    d, toks, ref, _ = model
    eng = make_engine(d, dtype, page_size=64, max_tokens=1024, max_requests=4)
    check_logits(step_all(eng, "w", toks, [200]), ref, dtype, "wide whole")
    eng.release("w")
    # a portion that ends inside a page, single tokens over a page's edge (captured steps), more portions
    got = step_all(eng, "p", toks, [60] + [1] * 10 + [100, 2, 28])
    check_logits(got, ref, dtype, "wide portions and single tokens")
    eng.release("p")


def _logits_at(plain, tokens, rows):
    """The plain implementation's logits at some places of a sequence (the head over a
    vocabulary of 65,536 is most of its time, so only where they are compared)."""
    import plain_lfm2 as P
    x = plain.hidden(tokens)[rows]
    return P.linear(P.rms_norm(x, plain.w["model.embedding_norm.weight"], plain.eps),
                    plain.w["model.embed_tokens.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("live", [24, 64, 100])
def test_many_decoding_requests_at_benchmark_width(wide, dtype, live):
    _many_decoding_requests(wide, dtype, live)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("live", [24, 100])
def test_many_decoding_requests_at_the_smaller_widths(narrower, dtype, live):
    _many_decoding_requests(narrower, dtype, live)


def _many_decoding_requests(model, dtype, live):
    """24, 64 and 100 live requests of different contexts decode six tokens each, every row held
    to the plain implementation: the step run launch by launch, the captured one and its
    replays. Beyond 16 rows the few-row products take more weight rows a block, the conv
    mixer takes two launches instead of the fused one, and the captured graph is another;
    beyond 64 rows the products go to the tile kernels, in slices of K."""
    from imparo_amd.engine import StepEntry
    d, _, _, plain = model
    rng = random.Random(live)
    contexts = [rng.randint(1, 90) for _ in range(live)]
    contexts[0], contexts[1], contexts[2] = 64, 63, 1            # a page's edge among them
    seqs = [prompt_tokens(65536, c + 6, 300 + i) for i, c in enumerate(contexts)]
    want = [_logits_at(plain, s, list(range(c, c + 6))) for s, c in zip(seqs, contexts)]
    eng = make_engine(d, dtype, page_size=64, max_tokens=live * 128, max_requests=live)
    for lo in range(0, live, 16):                                 # prompts, sixteen requests a step
        eng.step([StepEntry(i, seqs[i][:contexts[i]], []) for i in range(lo, min(live, lo + 16))])
    for j in range(6):
        out = eng.step([StepEntry(i, [seqs[i][contexts[i] + j]], [0]) for i in range(live)]).cpu()
        ref = torch.stack([w[j] for w in want])
        check_logits(out, ref, dtype, f"{live} decoding rows, step {j}")
    assert not eng.use_graphs or len(eng._graphs) == 1           # steps 1.. ran from one captured graph
    for i in range(live):
        eng.release(i)
    assert eng.free_pages() == [eng.cache.groups[0].pool.n_pages]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_at_benchmark_width_with_pages_used_again(wide, dtype):
    """Up to four live requests, portions of some beside decoded tokens of others, pages of 64
    and a pool no larger than the schedule's peak, so that later requests get earlier ones' pages."""
    from imparo_amd.engine import StepEntry
    d, _, _, plain = wide
    rng = random.Random(5)
    lengths = [150, 70, 200, 40, 130, 90, 65]
    prompts = [prompt_tokens(65536, n, 400 + i) for i, n in enumerate(lengths)]
    steps = mixed_schedule(rng, lengths, sizes=(1, 1, 1, 2, 3, 17, 40, 64, 100))
    pool = peak_pages(steps, 64)
    assert sum((n + 63) // 64 for n in lengths) > pool
    eng = make_engine(d, dtype, page_size=64, max_tokens=pool * 64, max_requests=4)
    got = {i: [] for i in range(len(lengths))}
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
    assert eng.free_pages() == [pool]
    for rid in range(len(lengths)):
        check_logits(torch.cat(got[rid]), plain.logits(prompts[rid]), dtype, f"wide mixed request {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("decoding", [24, 40])
def test_many_decoding_rows_beside_portions_in_one_step(wide, dtype, decoding):
    """24 and 40 requests bring one token each beside a 33-token and a 300-token portion of two
    others, all in one step, three steps in a row. With more than 16 single-token rows beside
    portions the attention mixer takes its two-launch form (head norm and cache write, then the
    split kernel for the single rows and the tiled one for the portions), the conv mixer its
    unfused one, and the products the 17-to-64-row or the tile kernels on 357 to 373 rows. Every
    row, single or of a portion, is held to the plain implementation."""
    from imparo_amd.engine import StepEntry
    d, _, _, plain = wide
    rng = random.Random(decoding)
    contexts = [rng.randint(1, 100) for _ in range(decoding)]
    contexts[0], contexts[1], contexts[2] = 64, 63, 1
    seqs = [prompt_tokens(65536, c + 3, 700 + i) for i, c in enumerate(contexts)]
    want = [_logits_at(plain, s, list(range(c, c + 3))) for s, c in zip(seqs, contexts)]
    # two prompts that come in portions: 33 + 33 + 33 and 300 + 300 + 100, the second over page edges
    short, longer = prompt_tokens(65536, 99, 801), prompt_tokens(65536, 700, 802)
    short_cuts, long_cuts = [(0, 33), (33, 66), (66, 99)], [(0, 300), (300, 600), (600, 700)]
    short_rows, long_rows = [5, 32, 33, 65, 66, 98], [0, 63, 64, 299, 300, 511, 512, 599, 600, 699]
    want_short, want_long = _logits_at(plain, short, short_rows), _logits_at(plain, longer, long_rows)
    pool_tokens = sum((c + 3 + 63) // 64 * 64 for c in contexts) + 128 + 704
    eng = make_engine(d, dtype, page_size=64, max_tokens=pool_tokens, max_requests=decoding + 2)
    for lo in range(0, decoding, 16):
        eng.step([StepEntry(i, seqs[i][:contexts[i]], []) for i in range(lo, min(decoding, lo + 16))])
    got_short, got_long = [], []
    for j in range(3):
        (slo, shi), (llo, lhi) = short_cuts[j], long_cuts[j]
        s_want = [r - slo for r in short_rows if slo <= r < shi]
        l_want = [r - llo for r in long_rows if llo <= r < lhi]
        entries = [StepEntry(i, [seqs[i][contexts[i] + j]], [0]) for i in range(decoding // 2)]
        entries.append(StepEntry("short", short[slo:shi], s_want))
        entries += [StepEntry(i, [seqs[i][contexts[i] + j]], [0]) for i in range(decoding // 2, decoding)]
        entries.append(StepEntry("long", longer[llo:lhi], l_want))
        out = eng.step(entries).cpu()
        half = decoding // 2
        rows_single = torch.cat([out[:half], out[half + len(s_want):half + len(s_want) + decoding - half]])
        got_short.append(out[half:half + len(s_want)])
        got_long.append(out[decoding + len(s_want):])
        check_logits(rows_single, torch.stack([w[j] for w in want]), dtype, f"{decoding} single rows beside portions, step {j}")
    check_logits(torch.cat(got_short), want_short, dtype, "the 33-token portions")
    check_logits(torch.cat(got_long), want_long, dtype, "the 300-token portions")
