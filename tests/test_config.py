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
                                 "num_attention_heads", "num_key_value_heads", "conv_L_cache", "block_ff_dim"])
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


# ---- the spellings checkpoints of this architecture carry: each works or is refused by name
def _without(d, *keys):
    return {k: v for k, v in d.items() if k not in keys}


def test_full_attn_idxs_stands_in_for_layer_types():
    d = dict(_without(TINY_B, "layer_types"), full_attn_idxs=[2, 4, 5])
    assert Lfm2Config.from_dict(d).layer_types == TINY_B["layer_types"]
    # both, agreeing, is fine; disagreeing or out of range is refused
    Lfm2Config.from_dict(dict(TINY_B, full_attn_idxs=[2, 4, 5]))
    with pytest.raises(Inconsistent, match="full_attn_idxs"):
        Lfm2Config.from_dict(dict(TINY_B, full_attn_idxs=[1, 4, 5]))
    with pytest.raises(Inconsistent, match="full_attn_idxs"):
        Lfm2Config.from_dict(dict(d, full_attn_idxs=[2, 9]))
    with pytest.raises(BadValue, match="full_attn_idxs"):
        Lfm2Config.from_dict(dict(d, full_attn_idxs="2,4,5"))
    with pytest.raises(MissingKey, match="layer_types.*full_attn_idxs"):
        Lfm2Config.from_dict(_without(TINY_B, "layer_types"))


def test_rope_theta_inside_rope_parameters():
    d = dict(_without(TINY_A, "rope_theta"), rope_parameters=dict(rope_theta=12345.0, rope_type="default"))
    cfg, plan = plan_from_config(d)
    assert cfg.rope_theta == 12345.0 and plan.layers[1].mixer["position"]["base"] == 12345.0
    Lfm2Config.from_dict(dict(TINY_A, rope_parameters=dict(rope_theta=10000.0)))          # said twice, agreeing
    with pytest.raises(Inconsistent, match="rope_theta"):
        Lfm2Config.from_dict(dict(TINY_A, rope_parameters=dict(rope_theta=12345.0)))
    with pytest.raises(BadValue, match="rope_type"):
        Lfm2Config.from_dict(dict(d, rope_parameters=dict(rope_theta=1e4, rope_type="yarn")))
    with pytest.raises(BadValue, match="factor"):
        Lfm2Config.from_dict(dict(d, rope_parameters=dict(rope_theta=1e4, factor=4.0)))
    with pytest.raises(BadValue, match="rope_scaling"):
        Lfm2Config.from_dict(dict(TINY_A, rope_scaling=dict(type="linear", factor=2.0)))
    assert Lfm2Config.from_dict(_without(TINY_A, "rope_theta")).rope_theta == 1000000.0  # the architecture's default


def test_tie_word_embeddings_is_read():
    d = dict(_without(TINY_A, "tie_embedding"), tie_word_embeddings=False)
    cfg, plan = plan_from_config(d)
    assert not cfg.tie_embedding and plan.head.prefix == "lm_head"
    assert plan_from_config(dict(d, tie_word_embeddings=True))[1].head.prefix == "model.embed_tokens"
    with pytest.raises(Inconsistent, match="tie_word_embeddings"):
        Lfm2Config.from_dict(dict(TINY_A, tie_word_embeddings=False))
    with pytest.raises(BadValue, match="tie_word_embeddings"):
        Lfm2Config.from_dict(dict(d, tie_word_embeddings="no"))


def test_eos_token_id_as_an_id_or_a_list():
    assert plan_from_config(dict(TINY_A, eos_token_id=7))[1].stop_token_ids == (7,)
    assert plan_from_config(dict(TINY_A, eos_token_id=[7, 2]))[1].stop_token_ids == (7, 2)
    assert plan_from_config(TINY_A)[1].stop_token_ids == ()
    for bad in ([], "7", [7, "2"], 7.0, True):
        with pytest.raises(BadValue, match="eos_token_id"):
            Lfm2Config.from_dict(dict(TINY_A, eos_token_id=bad))
    with pytest.raises(Inconsistent, match="eos_token_id"):
        Lfm2Config.from_dict(dict(TINY_A, eos_token_id=[7, 256]))


def test_feed_forward_width_keys():
    base = _without(TINY_B, "block_ff_dim", "block_auto_adjust_ff_dim")
    # intermediate_size alone is the width before adjustment; adjustment is on unless the file says otherwise
    assert Lfm2Config.from_dict(dict(base, intermediate_size=480)).ff_dim == 320
    assert Lfm2Config.from_dict(dict(base, intermediate_size=480, block_auto_adjust_ff_dim=False)).ff_dim == 480
    # block_ff_dim wins where a file carries both
    assert Lfm2Config.from_dict(dict(base, intermediate_size=1000, block_ff_dim=480)).ff_dim == 320
    assert Lfm2Config.from_dict(dict(base, intermediate_size=1000, block_ff_dim=480,
                                     block_auto_adjust_ff_dim=False)).ff_dim == 480
    with pytest.raises(MissingKey, match="block_ff_dim.*intermediate_size"):
        Lfm2Config.from_dict(base)


def test_restated_and_unsupported_keys_are_refused_and_unknown_ones_are_listed():
    full = dict(TINY_A, block_dim=64, conv_dim=64, conv_dim_out=64, num_heads=4, block_norm_eps=1e-5, theta=10000.0,
                block_use_swiglu=True, use_pos_enc=True, torch_dtype="bfloat16", bos_token_id=1, pad_token_id=0,
                use_cache=True, initializer_range=0.02, transformers_version="x", block_mlp_init_scale=1.0)
    assert Lfm2Config.from_dict(full).unread_keys == []
    for key, value in (("block_dim", 128), ("conv_dim", 32), ("conv_dim_out", 32), ("num_heads", 8),
                       ("block_norm_eps", 1e-6), ("theta", 5.0)):
        with pytest.raises(Inconsistent, match=key):
            Lfm2Config.from_dict(dict(full, **{key: value}))
    for key, value in (("block_use_swiglu", False), ("use_pos_enc", False)):
        with pytest.raises(BadValue, match=key):
            Lfm2Config.from_dict(dict(full, **{key: value}))
    assert Lfm2Config.from_dict(dict(full, some_new_switch=3)).unread_keys == ["some_new_switch"]


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
