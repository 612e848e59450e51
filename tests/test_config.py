"""Configuration: typed reading of config.json, the four error classes, the
registry, and the plan derived from a configuration."""
import copy

import pytest

from imparo_amd.config import (Lfm2Config, plan_from_config, known_architectures, register_architecture,
                               UnknownArchitecture, MissingKey, BadValue, Inconsistent, adjusted_ff_dim)
from tiny_configs import TINY_A, TINY_B, TINY_C


def test_reads_every_key_and_derives_sizes():
    a = Lfm2Config.from_dict(TINY_A)
    assert (a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (64, 4, 2, 16)
    assert a.ff_dim == 192 and a.conv_L_cache == 3 and not a.conv_bias and a.tie_embedding
    assert a.rope_theta == 10000.0 and a.norm_eps == 1e-5
    b = Lfm2Config.from_dict(TINY_B)
    assert b.head_dim == 32 and b.ff_dim == 320 and b.conv_bias and not b.tie_embedding
    assert b.layer_types.count("conv") == 3 and b.norm_eps == 1e-6
    c = Lfm2Config.from_dict(TINY_C)
    assert c.sliding_window == 24 and c.head_dim == 16


def test_ff_dim_adjustment_matches_the_published_shapes():
    assert adjusted_ff_dim(12288, 256, 1.0) == 8192
    assert adjusted_ff_dim(10240, 256, 1.0) == 6912
    assert adjusted_ff_dim(6656, 256, 1.0) == 4608
    assert adjusted_ff_dim(480, 64, 1.0) == 320
    assert adjusted_ff_dim(480, 64, None) == 320
    assert adjusted_ff_dim(480, 64, 1.5) == 512      # int(1.5 * 320) = 480 -> next multiple of 64


def test_benchmark_shape():
    cfg = dict(TINY_A, vocab_size=65536, hidden_size=2048, num_hidden_layers=16, num_attention_heads=32,
               num_key_value_heads=8, block_auto_adjust_ff_dim=True, block_ff_dim=12288, block_multiple_of=256,
               layer_types=["full_attention" if i in (2, 5, 8, 10, 12, 14) else "conv" for i in range(16)])
    c = Lfm2Config.from_dict(cfg)
    assert c.head_dim == 64 and c.ff_dim == 8192


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers", "layer_types",
                                 "num_attention_heads", "num_key_value_heads", "conv_L_cache"])
def test_missing_key(key):
    d = copy.deepcopy(TINY_A)
    del d[key]
    with pytest.raises(MissingKey, match=key):
        Lfm2Config.from_dict(d)


def test_bad_values():
    for key, value in (("hidden_size", "64"), ("vocab_size", 0), ("conv_bias", 1), ("norm_eps", "tiny"),
                       ("layer_types", "conv"), ("num_hidden_layers", 4.0), ("sliding_window", 0)):
        with pytest.raises(BadValue, match=key):
            Lfm2Config.from_dict(dict(TINY_A, **{key: value}))
    with pytest.raises(BadValue, match="layer_types\\[1\\]"):
        Lfm2Config.from_dict(dict(TINY_A, layer_types=["conv", "mamba", "conv", "full_attention"]))


def test_inconsistent():
    with pytest.raises(Inconsistent, match="layer_types has 4 entries"):
        Lfm2Config.from_dict(dict(TINY_A, num_hidden_layers=5))
    with pytest.raises(Inconsistent, match="not a multiple"):
        Lfm2Config.from_dict(dict(TINY_A, num_attention_heads=5))
    with pytest.raises(Inconsistent, match="num_key_value_heads"):
        Lfm2Config.from_dict(dict(TINY_A, num_key_value_heads=3))
    with pytest.raises(Inconsistent, match="at least 2 taps"):
        Lfm2Config.from_dict(dict(TINY_A, conv_L_cache=1))
    with pytest.raises(Inconsistent, match="sliding_window"):
        Lfm2Config.from_dict(dict(TINY_A, layer_types=["conv", "sliding_attention", "conv", "full_attention"]))


def test_registry():
    assert "Lfm2ForCausalLM" in known_architectures()
    with pytest.raises(UnknownArchitecture, match="Lfm2ForCausalLM"):   # the error lists what is known
        plan_from_config(dict(TINY_A, architectures=["LlamaForCausalLM"]))
    with pytest.raises(MissingKey):
        plan_from_config({k: v for k, v in TINY_A.items() if k != "architectures"})


def test_plan_is_chosen_layer_by_layer():
    _, plan = plan_from_config(TINY_C)
    kinds = [l.mixer.kind for l in plan.layers]
    assert kinds == ["attention", "short_conv", "attention", "attention", "short_conv"]
    assert [l.mixer.get("window") for l in plan.layers] == [24, None, None, 24, None]
    assert all(l.ffn.kind == "swiglu" and l.ffn["hidden"] == 172 for l in plan.layers)
    assert [c.layer for c in plan.order] == [0, 1, 2, 3, 4] and all(c.cache_of is None for c in plan.order)
    assert plan.layers[0].mixer["position"]["base"] == 50000.0
    assert plan.layers[0].mixer_norm["eps"] == 1e-4
    _, b = plan_from_config(TINY_B)
    assert b.head.prefix == "lm_head" and b.layers[0].mixer["bias"] and b.layers[0].mixer["taps"] == 4
    _, a = plan_from_config(TINY_A)
    assert a.head.prefix == "model.embed_tokens"


def test_plan_order_is_validated():
    from imparo_amd.config import LayerCall
    import dataclasses
    _, plan = plan_from_config(TINY_A)
    bad = dataclasses.replace(plan, order=[LayerCall(0), LayerCall(7)])
    with pytest.raises(Inconsistent):
        bad.validate()
    bad = dataclasses.replace(plan, order=[LayerCall(1, cache_of=0)])
    with pytest.raises(Inconsistent):
        bad.validate()
    ok = dataclasses.replace(plan, order=[LayerCall(0), LayerCall(1), LayerCall(1, cache_of=1), LayerCall(0)])
    ok.validate()
