"""Weights: the safetensors container, loading by name with one clear error,
and the random-weights mode."""
import json
import os

import pytest
import torch

from imparo_amd import write_random_model, WeightsError
from imparo_amd.config import plan_from_config
from imparo_amd.engine.model import declared_tensors
from imparo_amd.weights import load_weights, save_file, SafetensorsFile, SafetensorsError
from tiny_configs import TINY_A, TINY_B, TINY_C, C_KEEP_F32


def _declared(cfg):
    _, plan = plan_from_config(cfg)
    return {k: d for k, (d, _) in declared_tensors(plan).items()}


def test_container_round_trip_and_agrees_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file as st_save
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.arange(7, dtype=torch.int32),
         "c": torch.randn(2, 2, 2), "empty": torch.zeros(0, 4)}
    p = str(tmp_path / "x.safetensors")
    save_file(t, p)
    theirs = load_file(p)                       # their reader, our writer
    for k in t:
        assert torch.equal(theirs[k], t[k]) and theirs[k].dtype == t[k].dtype
    p2 = str(tmp_path / "y.safetensors")
    st_save(t, p2)                              # their writer, our reader
    f = SafetensorsFile(p2)
    for k in t:
        assert torch.equal(f.tensor(k), t[k]) and f.dtype(k) == t[k].dtype
    f.close()


def test_container_rejects_garbage(tmp_path):
    p = tmp_path / "bad.safetensors"
    p.write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00not json at all!!")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(p))
    p.write_bytes(b"\xff\xff\xff\xff\xff\xff\xff\x7f{}")
    with pytest.raises(SafetensorsError, match="exceeds"):
        SafetensorsFile(str(p))


def test_declared_names_are_the_architecture_s_own():
    names = set(_declared(TINY_B))
    assert "model.embed_tokens.weight" in names and "lm_head.weight" in names
    assert "model.embedding_norm.weight" in names
    assert {"model.layers.0.conv.in_proj.weight", "model.layers.0.conv.conv.weight", "model.layers.0.conv.out_proj.bias",
            "model.layers.0.operator_norm.weight", "model.layers.0.ffn_norm.weight",
            "model.layers.2.self_attn.q_proj.weight", "model.layers.2.self_attn.k_layernorm.weight",
            "model.layers.2.self_attn.out_proj.weight", "model.layers.2.feed_forward.w1.weight",
            "model.layers.2.feed_forward.w3.weight", "model.layers.2.feed_forward.w2.weight"} <= names
    # only the arm a layer's kind needs
    assert not any(n.startswith("model.layers.0.self_attn") for n in names)
    assert not any(n.startswith("model.layers.2.conv") for n in names)
    a = _declared(TINY_A)
    assert "lm_head.weight" not in a and a["model.layers.0.conv.conv.weight"].shape == (64, 1, 3)
    assert "model.layers.0.conv.in_proj.bias" not in a


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = str(tmp_path / "m")
    write_random_model(TINY_A, 0, d)
    from safetensors.torch import load_file
    t = load_file(os.path.join(d, "model.safetensors"))
    del t["model.layers.1.self_attn.q_layernorm.weight"]
    del t["model.embedding_norm.weight"]
    t["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 64, dtype=torch.bfloat16)   # a conv layer
    t["model.layers.2.feed_forward.w2.weight"] = torch.zeros(192, 64, dtype=torch.bfloat16)   # transposed
    t["model.layers.3.ffn_norm.weight"] = torch.zeros(64, dtype=torch.int32)
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_weights(d, _declared(TINY_A))
    msg = str(e.value)
    assert e.value.missing == ["model.embedding_norm.weight", "model.layers.1.self_attn.q_layernorm.weight"]
    assert e.value.unexpected == ["model.layers.0.self_attn.q_proj.weight"]
    assert "model.layers.2.feed_forward.w2.weight is [192, 64], expected [64, 192]" in msg
    assert "unsupported dtype: model.layers.3.ffn_norm.weight" in msg
    for name in e.value.missing + e.value.unexpected:
        assert name in msg


def test_storage_dtypes(tmp_path):
    d = str(tmp_path / "c")
    write_random_model(TINY_C, 2, d, keep_float32=C_KEEP_F32)
    w = load_weights(d, _declared(TINY_C))
    assert w["model.layers.0.operator_norm.weight"].dtype == torch.float32        # stored in 32 bits: stays
    assert w["model.layers.1.conv.in_proj.weight"].dtype == torch.float32
    assert w["model.layers.1.conv.out_proj.weight"].dtype == torch.bfloat16
    # float16 in the file is kept in bfloat16
    from safetensors.torch import load_file
    t = load_file(os.path.join(d, "model.safetensors"))
    t["model.layers.1.conv.out_proj.weight"] = t["model.layers.1.conv.out_proj.weight"].to(torch.float16)
    save_file(t, os.path.join(d, "model.safetensors"))
    assert load_weights(d, _declared(TINY_C))["model.layers.1.conv.out_proj.weight"].dtype == torch.bfloat16


def test_random_mode_is_seeded_and_has_the_stated_spreads(tmp_path):
    a1, a2, a3 = str(tmp_path / "1"), str(tmp_path / "2"), str(tmp_path / "3")
    write_random_model(TINY_B, 1, a1)
    write_random_model(TINY_B, 1, a2)
    write_random_model(TINY_B, 2, a3)
    w1, w2, w3 = (load_weights(x, _declared(TINY_B)) for x in (a1, a2, a3))
    for k in _declared(TINY_B):
        assert torch.equal(w1[k], w2[k])
    assert not torch.equal(w1["lm_head.weight"], w3["lm_head.weight"])
    assert json.load(open(os.path.join(a1, "config.json")))["hidden_size"] == 96
    assert abs(w1["lm_head.weight"].float().std().item() - 0.02) < 0.002
    assert abs(w1["model.layers.0.conv.conv.weight"].float().std().item() - 0.1) < 0.03
    n = w1["model.layers.0.operator_norm.weight"].float()
    assert 0.9 <= n.min() and n.max() <= 1.1 and abs(n.mean().item() - 1.0) < 0.03
    assert abs(w1["model.layers.0.conv.in_proj.bias"].float().std().item() - 0.02) < 0.005


def test_a_sharded_checkpoint_is_read_through_its_index(tmp_path):
    d = str(tmp_path / "whole")
    write_random_model(TINY_B, 1, d)
    whole = load_weights(d, _declared(TINY_B))
    names = sorted(_declared(TINY_B))
    s = str(tmp_path / "sharded")
    os.makedirs(s)
    parts = {"model-00001-of-00003.safetensors": names[0::3], "model-00002-of-00003.safetensors": names[1::3],
             "model-00003-of-00003.safetensors": names[2::3]}
    for shard, held in parts.items():
        save_file({n: whole[n] for n in held}, os.path.join(s, shard))
    index = {"metadata": {}, "weight_map": {n: shard for shard, held in parts.items() for n in held}}
    with open(os.path.join(s, "model.safetensors.index.json"), "w") as f:
        json.dump(index, f)
    got = load_weights(s, _declared(TINY_B))
    for n in names:
        assert torch.equal(got[n], whole[n])
    # faults of a sharded folder come in the same one error, named after the index
    del index["weight_map"][names[4]]
    held = [n for n in parts["model-00002-of-00003.safetensors"] if n != names[4]]
    save_file({n: whole[n] for n in held}, os.path.join(s, "model-00002-of-00003.safetensors"))
    with open(os.path.join(s, "model.safetensors.index.json"), "w") as f:
        json.dump(index, f)
    with pytest.raises(WeightsError, match="index.json") as e:
        load_weights(s, _declared(TINY_B))
    assert e.value.missing == [names[4]]
    # a shard the index names but the folder lacks
    os.remove(os.path.join(s, "model-00003-of-00003.safetensors"))
    with pytest.raises(FileNotFoundError, match="model-00003-of-00003"):
        load_weights(s, _declared(TINY_B))
    with pytest.raises(FileNotFoundError, match="neither"):
        load_weights(str(tmp_path), _declared(TINY_B))


def test_a_stored_head_beside_a_tied_embedding_must_equal_it(tmp_path):
    from imparo_amd.config import plan_from_config
    d = str(tmp_path / "m")
    write_random_model(TINY_A, 0, d)
    _, plan = plan_from_config(TINY_A)
    assert plan.restated_tensors == {"lm_head.weight": "model.embed_tokens.weight"}
    from safetensors.torch import load_file
    t = load_file(os.path.join(d, "model.safetensors"))
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError) as e:          # nobody said what it may restate
        load_weights(d, _declared(TINY_A))
    assert e.value.unexpected == ["lm_head.weight"]
    w = load_weights(d, _declared(TINY_A), plan.restated_tensors)
    assert "lm_head.weight" not in w
    t["lm_head.weight"][3, 5] += 1.0
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_weights(d, _declared(TINY_A), plan.restated_tensors)
    assert e.value.unexpected == ["lm_head.weight"]
    # an untied model has no such allowance: it declares its head
    assert plan_from_config(TINY_B)[1].restated_tensors == {}


def test_offsets_that_overlap_or_run_backwards_are_refused(tmp_path):
    import struct
    def write(path, header, n_bytes):
        blob = json.dumps(header).encode()
        with open(path, "wb") as f:
            f.write(struct.pack("<Q", len(blob)) + blob + b"\0" * n_bytes)
    p = str(tmp_path / "x.safetensors")
    write(p, {"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
              "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, 12)
    with pytest.raises(SafetensorsError, match="overlap"):
        SafetensorsFile(p)
    write(p, {"a": {"dtype": "F32", "shape": [2], "data_offsets": [-8, 0]}}, 8)
    with pytest.raises(SafetensorsError, match="inconsistent offsets"):
        SafetensorsFile(p)
