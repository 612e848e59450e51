"""Layers of the benchmark's own width (hidden 2048, 32 heads of 64 over 8 kv
heads, feed-forward 8192, vocabulary 65536) with few layers, so that the plain
implementation can follow on the CPU: the kernels' paths for these sizes (the
128x128 MFMA tiles, the wide few-row products, the float4 norm, matrix-core
attention at head size 64, pages of 64) are compared end to end."""
import pytest
import torch

from conftest import prompt_tokens
from gpu_helpers import make_engine, step_all
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


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    from imparo_amd import write_random_model
    from plain_lfm2 import PlainLfm2
    d = str(tmp_path_factory.mktemp("wide"))
    write_random_model(WIDE, 2, d)
    plain = PlainLfm2(d)
    toks = prompt_tokens(65536, 200, 77)
    return d, toks, plain.logits(toks)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_benchmark_width_layers(wide, dtype):
    d, toks, ref = wide
    eng = make_engine(d, dtype, page_size=64, max_tokens=1024, max_requests=4)
    check_logits(step_all(eng, "w", toks, [200]), ref, dtype, "wide whole")
    eng.release("w")
    # a portion that ends inside a page, single tokens over a page's edge (captured steps), more portions
    got = step_all(eng, "p", toks, [60] + [1] * 10 + [100, 2, 28])
    check_logits(got, ref, dtype, "wide portions and single tokens")
    eng.release("p")
