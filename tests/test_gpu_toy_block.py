"""Another arrangement of a block and another pairing of rotated dimensions,
defined here and registered without a change to the framework's files. They
are no model of anyone's.

Sandwich block: three norms instead of two,
    x += post_norm( mixer( mixer_norm(x) ) );   x += ffn( ffn_norm(x) )
with the third norm's weight a tensor of its own. The plan names the block's
parts; the builder and the loader walk them without knowing which they are.

Interleaved rotation: pair i is dimensions (2i, 2i + 1) instead of
(i, i + half); the position part only says so, the kernel takes it as an
argument.
"""
import dataclasses
import math

import numpy as np
import pytest
import torch

from conftest import prompt_tokens
from tolerances import check_logits

pytestmark = pytest.mark.gpu

ROTARY_BASE = 300.0


class SandwichBlock:
    """The block interface: __init__(parts by name), cache_spec(page_size),
    forward(ctx, residual, site, owns_cache)."""
    role = "block"
    graph_safe = True         # launches kernels only

    def __init__(self, parts):
        self.mixer_norm, self.mixer, self.post_norm = parts["mixer_norm"], parts["mixer"], parts["mixer_post_norm"]
        self.ffn_norm, self.ffn = parts["ffn_norm"], parts["ffn"]

    def cache_spec(self, page_size):
        return self.mixer.cache_spec(page_size)

    def forward(self, ctx, res, site, owns_cache):
        from imparo_amd.parts.base import Residual
        h = self.mixer_norm.forward(ctx, res, self.mixer.in_dtype)
        m = self.mixer.forward(ctx, site, owns_cache, h)
        # the mixer's output may come as slices of its last product's inner dimension: the norm adds them up
        inner = Residual(m[0], m[1:]) if m.dim() == 3 and m.shape[0] > 1 else Residual(m[0] if m.dim() == 3 else m)
        res.pending = self.post_norm.forward(ctx, inner, torch.float32, name="post_normed")
        n = self.ffn_norm.forward(ctx, res, self.ffn.in_dtype)
        res.pending = self.ffn.forward(ctx, n)


class InterleavedRope:
    """The position interface: rotary_dim, inv_freq, and which dimensions pair."""
    role = "position"
    interleaved = True

    def __init__(self, spec, device):
        self.rotary_dim = int(spec["rotary_dim"])
        self.inv_freq = torch.from_numpy(inv_freq(self.rotary_dim, float(spec["base"]))).to(device)


def inv_freq(rot, base):
    i = np.arange(rot // 2, dtype=np.float32)
    return np.power(np.float32(base), (np.float32(-2.0) * i / np.float32(rot)).astype(np.float32)).astype(np.float32)


def plain_rotate_interleaved(x, positions, rot):
    theta = (np.asarray(positions, dtype=np.float64)[:, None] * inv_freq(rot, ROTARY_BASE).astype(np.float64)
             ).astype(np.float32)
    cos, sin = (torch.from_numpy(f(theta)).unsqueeze(1) for f in (np.cos, np.sin))
    out = x.clone()
    x0, x1 = x[..., 0:rot:2], x[..., 1:rot:2]
    out[..., 0:rot:2] = x0 * cos - x1 * sin
    out[..., 1:rot:2] = x0 * sin + x1 * cos
    return out


@pytest.fixture(scope="module")
def sandwich(tmp_path_factory):
    from imparo_amd import register_part, register_architecture, write_random_model, PartSpec
    from imparo_amd.config import Lfm2Config, LayerPlan, lfm2
    register_part("block", "test_sandwich", SandwichBlock)
    register_part("position", "test_interleaved_rope", InterleavedRope)

    def build(cfg):
        plan = lfm2.build_plan(cfg)
        layers = []
        for i, layer in enumerate(plan.layers):
            if layer.mixer.kind == "attention":
                params = dict(layer.mixer.params)
                params["position"] = PartSpec("test_interleaved_rope", "", dict(rotary_dim=cfg.head_dim, base=ROTARY_BASE))
                layer = layer.with_part("mixer", PartSpec(layer.mixer.kind, layer.mixer.prefix, params))
            third = PartSpec("rms_norm", f"model.layers.{i}.post_mixer_norm", dict(width=cfg.hidden_size, eps=cfg.norm_eps))
            layer = layer.with_part("mixer_post_norm", third, role="norm")
            layers.append(LayerPlan(layer.parts, "test_sandwich"))
        return dataclasses.replace(plan, architecture="TestSandwichForCausalLM", layers=layers)
    register_architecture("TestSandwichForCausalLM", Lfm2Config.from_dict, build)
    from tiny_configs import TINY_B
    cfg = dict(TINY_B, architectures=["TestSandwichForCausalLM"])
    d = str(tmp_path_factory.mktemp("sandwich"))
    write_random_model(cfg, 21, d, layer_gain=4.0)
    return d, cfg


def plain_logits(model_dir, cfg, tokens):
    from plain_lfm2 import PlainLfm2, rms_norm, swiglu, linear, attend
    m = PlainLfm2(model_dir)
    T = len(tokens)
    positions = np.arange(T)
    x = m.w["model.embed_tokens.weight"][torch.as_tensor(tokens)]
    for i, kind in enumerate(cfg["layer_types"]):
        p = f"model.layers.{i}."
        h = rms_norm(x, m.w[p + "operator_norm.weight"], m.eps)
        if kind == "conv":
            mix = m.mixer_conv(i, h)
        else:
            a = p + "self_attn."
            q = linear(h, m.w[a + "q_proj.weight"]).reshape(T, m.H, m.D)
            k = linear(h, m.w[a + "k_proj.weight"]).reshape(T, m.Hk, m.D)
            v = linear(h, m.w[a + "v_proj.weight"]).reshape(T, m.Hk, m.D)
            q = plain_rotate_interleaved(rms_norm(q, m.w[a + "q_layernorm.weight"], m.eps), positions, m.D)
            k = plain_rotate_interleaved(rms_norm(k, m.w[a + "k_layernorm.weight"], m.eps), positions, m.D)
            o = attend(q, k, v, positions, 1.0 / math.sqrt(m.D), None)
            mix = linear(o.reshape(T, m.H * m.D), m.w[a + "out_proj.weight"])
        x = x + rms_norm(mix, m.w[p + "post_mixer_norm.weight"], m.eps)
        n = rms_norm(x, m.w[p + "ffn_norm.weight"], m.eps)
        x = x + swiglu(n, m.w[p + "feed_forward.w1.weight"], m.w[p + "feed_forward.w3.weight"],
                       m.w[p + "feed_forward.w2.weight"])
    return linear(rms_norm(x, m.w["model.embedding_norm.weight"], m.eps), m.w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_block_with_a_third_norm_is_built_and_stepped(sandwich, dtype):
    from imparo_amd.engine import Engine, StepEntry, declared_tensors
    d, cfg = sandwich
    eng = Engine(d, dtype=dtype, max_tokens=512, page_size=16, max_requests=3)
    assert all(type(b).__name__ == "SandwichBlock" for b in eng.model.blocks)
    assert "model.layers.3.post_mixer_norm.weight" in declared_tensors(eng.plan)      # the loader asked for it
    assert eng.model.graph_safe
    vocab = cfg["vocab_size"]
    a, b = prompt_tokens(vocab, 44, 1), prompt_tokens(vocab, 23, 2)
    out_a = [eng.step([StepEntry("a", a[:19], list(range(19)))]).cpu()]
    o = eng.step([StepEntry("a", a[19:21], [0, 1]), StepEntry("b", b[:16], list(range(16)))]).cpu()
    out_a.append(o[:2])
    out_b = [o[2:]]
    for i in range(21, 44):                      # a decodes (captured steps too) while b goes on one token at a time
        entries = [StepEntry("a", a[i:i + 1], [0])]
        j = 16 + (i - 21)
        if j < 23:
            entries.append(StepEntry("b", b[j:j + 1], [0]))
        o = eng.step(entries).cpu()
        out_a.append(o[:1])
        if j < 23:
            out_b.append(o[1:])
    check_logits(torch.cat(out_a), plain_logits(d, cfg, a), dtype, "sandwich a")
    check_logits(torch.cat(out_b), plain_logits(d, cfg, b), dtype, "sandwich b")


def test_interleaved_pairs_differ_from_halves():
    """The pairing is no detail: the same rows rotated as pairs (2i, 2i + 1) and as pairs
    (i, i + half) differ; both keep a pair's length and leave position 0 alone."""
    from plain_lfm2 import rope_neox
    q = torch.randn(6, 3, 32, generator=torch.Generator().manual_seed(1))
    a = plain_rotate_interleaved(q, np.arange(6), 32)
    b = rope_neox(q, np.arange(6), ROTARY_BASE, 32)
    assert (a - b).abs().max() > 0.1
    torch.testing.assert_close(a.norm(dim=-1), q.norm(dim=-1), rtol=1e-5, atol=1e-5)
    assert torch.equal(a[0], q[0])
