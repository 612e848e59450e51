"""A toy mixer with state of its own, defined here, is registered, built and
stepped without a change to the framework's files: a new part kind, a new
architecture name, random weights for it, the cache manager's slots for its
state, the step function, the scheduler.

The toy: a leaky running mean per channel, s_t = a * s_{t-1} + (1 - a) * (W h_t),
out_t = U s_t, with the decay `a` from the configuration and s kept per request
in a fixed-size slot. It is no model of anyone's.
"""
import json
import os

import pytest
import torch

from conftest import prompt_tokens
from tolerances import check_logits

pytestmark = pytest.mark.gpu


class LeakyMean:
    """The mixer interface: declare(spec), __init__(spec, tensors, device,
    engine_dtype), in_dtype, cache_spec(page_size), forward(ctx, site, owns_cache, h)."""
    role = "mixer"

    @staticmethod
    def declare(spec):
        from imparo_amd.weights import TensorDecl
        E = spec["width"]
        return {f"{spec.prefix}.w.weight": (TensorDecl((E, E)), "matrix"),
                f"{spec.prefix}.u.weight": (TensorDecl((E, E)), "matrix")}

    def __init__(self, spec, tensors, device, engine_dtype):
        from imparo_amd.parts import Linear, place_matrix
        self.width, self.decay = spec["width"], float(spec["decay"])
        self.w = Linear(place_matrix(tensors[f"{spec.prefix}.w.weight"], engine_dtype, device))
        self.u = Linear(place_matrix(tensors[f"{spec.prefix}.u.weight"], engine_dtype, device))

    @property
    def in_dtype(self):
        return self.w.in_dtype

    def cache_spec(self, page_size):
        from imparo_amd.cache import FixedSpec
        return FixedSpec((self.width,))

    def forward(self, ctx, site, owns_cache, h):
        z = self.w(ctx, h, torch.float32, "toy_z")
        state = ctx.fixed_state(site)                       # [slots, width] float32
        out = torch.empty_like(z)
        starts, lens, slots = ctx.seg_start.tolist(), ctx.seg_len.tolist(), ctx.slot.tolist()
        for start, n, slot in zip(starts, lens, slots):     # a scan per request: toy speed
            s = state[slot].clone()
            for t in range(start, start + n):
                s = self.decay * s + (1.0 - self.decay) * z[t]
                out[t] = s
            state[slot] = s
        return self.u(ctx, out.to(self.u.in_dtype), torch.float32, "mixer_out")


class LeakyMeanThatCounts(LeakyMean):
    """The same mixer keeping two tensors of fixed size per request, of different shapes and dtypes:
    its running mean in float32 and, in bfloat16, how many tokens the request has fed so far."""

    def cache_spec(self, page_size):
        from imparo_amd.cache import FixedArray, FixedSpec
        return FixedSpec(arrays=(FixedArray("mean", (self.width,)), FixedArray("fed", (2,), "bfloat16")))

    def forward(self, ctx, site, owns_cache, h):
        arrays = ctx.fixed_arrays(site)
        z = self.w(ctx, h, torch.float32, "toy_z")
        out = torch.empty_like(z)
        for start, n, slot in zip(ctx.seg_start.tolist(), ctx.seg_len.tolist(), ctx.slot.tolist()):
            s = arrays["mean"][slot].clone()
            for t in range(start, start + n):
                s = self.decay * s + (1.0 - self.decay) * z[t]
                out[t] = s
            arrays["mean"][slot] = s
            arrays["fed"][slot, 0] += n
        return self.u(ctx, out.to(self.u.in_dtype), torch.float32, "mixer_out")


def plain_leaky(h, w, u, decay):
    z = h @ w.t()
    s = torch.zeros(h.shape[1])
    out = []
    for t in range(h.shape[0]):
        s = decay * s + (1 - decay) * z[t]
        out.append(s)
    return torch.stack(out) @ u.t()


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from imparo_amd import register_part, register_architecture, write_random_model, PartSpec
    from imparo_amd.config import Lfm2Config, LayerPlan, LayerCall
    from imparo_amd.config import lfm2
    import dataclasses
    register_part("mixer", "test_leaky_mean", LeakyMean)

    def read(d):
        cfg = Lfm2Config.from_dict({k: v for k, v in d.items() if k not in ("toy_layers", "toy_decay")})
        cfg.toy_layers, cfg.toy_decay = d["toy_layers"], d["toy_decay"]
        return cfg

    def build(cfg):
        plan = lfm2.build_plan(cfg)
        layers = list(plan.layers)
        for i in cfg.toy_layers:
            toy = PartSpec("test_leaky_mean", f"model.layers.{i}.toy", dict(width=cfg.hidden_size, decay=cfg.toy_decay))
            layers[i] = layers[i].with_part("mixer", toy)
        return dataclasses.replace(plan, architecture="TestLeakyForCausalLM", layers=layers)
    register_architecture("TestLeakyForCausalLM", read, build)
    from tiny_configs import TINY_A
    cfg = dict(TINY_A, architectures=["TestLeakyForCausalLM"], toy_layers=[0, 3], toy_decay=0.75)
    d = str(tmp_path_factory.mktemp("toy"))
    write_random_model(cfg, 9, d)
    return d, cfg


def plain_toy_logits(model_dir, cfg, tokens):
    """The plain model with layers 0 and 3 replaced by the toy's formula."""
    from plain_lfm2 import PlainLfm2, rms_norm, swiglu, linear
    import numpy as np
    m = PlainLfm2(model_dir)
    x = m.w["model.embed_tokens.weight"][torch.as_tensor(tokens)]
    for i, kind in enumerate(cfg["layer_types"]):
        p = f"model.layers.{i}."
        h = rms_norm(x, m.w[p + "operator_norm.weight"], m.eps)
        if i in cfg["toy_layers"]:
            mix = plain_leaky(h, m.w[p + "toy.w.weight"], m.w[p + "toy.u.weight"], cfg["toy_decay"])
        elif kind == "conv":
            mix = m.mixer_conv(i, h)
        else:
            mix, _ = m.mixer_attention(i, h, np.arange(len(tokens)), None)
        x = x + mix
        n = rms_norm(x, m.w[p + "ffn_norm.weight"], m.eps)
        x = x + swiglu(n, m.w[p + "feed_forward.w1.weight"], m.w[p + "feed_forward.w3.weight"], m.w[p + "feed_forward.w2.weight"])
    return linear(rms_norm(x, m.w["model.embedding_norm.weight"], m.eps), m.w["model.embed_tokens.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_is_built_and_stepped(toy, dtype):
    from imparo_amd.engine import Engine, StepEntry
    from imparo_amd.cache import FixedSpec
    d, cfg = toy
    eng = Engine(d, dtype=dtype, max_tokens=512, page_size=8, max_requests=3)
    # layer 0 (was conv) and 3 (was attention) hold the toy's state; 2 keeps its conv state; 1 its pages
    assert [type(s).__name__ for s in eng.model.site_specs] == ["FixedSpec", "PagedSpec", "FixedSpec", "FixedSpec"]
    assert eng.model.site_specs[0] == FixedSpec((64,)) and len(eng.cache.groups) == 1
    a, b = prompt_tokens(256, 45, 1), prompt_tokens(256, 30, 2)
    ref_a, ref_b = plain_toy_logits(d, cfg, a), plain_toy_logits(d, cfg, b)
    out = []
    out.append(eng.step([StepEntry("a", a[:20], list(range(20)))]).cpu())
    o = eng.step([StepEntry("a", a[20:22], [0, 1]), StepEntry("b", b[:17], list(range(17)))]).cpu()
    out.append(o[:2])
    got_b = [o[2:]]
    for i in range(22, 45):                      # a decodes while b goes on in small portions
        entries = [StepEntry("a", a[i:i + 1], [0])]
        j = 17 + (i - 22)
        if j < 30:
            entries.append(StepEntry("b", b[j:j + 1], [0]))
        o = eng.step(entries).cpu()
        out.append(o[:1])
        if j < 30:
            got_b.append(o[1:])
    check_logits(torch.cat(out), ref_a, dtype, "toy a")
    check_logits(torch.cat(got_b), ref_b, dtype, "toy b")
    eng.release("a"), eng.release("b")
    # a slot that is used again starts from zero state
    again = eng.step([StepEntry("c", b, list(range(30)))]).cpu()
    check_logits(again, ref_b, dtype, "toy slot reuse")


def test_toy_model_generates_through_the_scheduler(toy):
    from imparo_amd import generate
    d, cfg = toy
    p = prompt_tokens(256, 11, 3)
    got = generate(d, [p], max_tokens=8, dtype="float32")[0]
    seq = list(p)
    for tok in got:
        assert int(torch.argmax(plain_toy_logits(d, cfg, seq)[-1])) == tok
        seq.append(tok)


def test_a_mixer_with_two_states_of_different_shape_and_dtype(toy, tmp_path):
    """The same model with the toy mixer keeping a float32 mean and a bfloat16 counter per request:
    both live in the request's slot, both start from zero when a slot is used again."""
    import dataclasses, shutil
    from imparo_amd import register_architecture, register_part, PartSpec
    from imparo_amd.config import Lfm2Config, lfm2
    from imparo_amd.engine import Engine, StepEntry
    d, cfg = toy
    register_part("mixer", "test_leaky_mean_counting", LeakyMeanThatCounts)

    def read(c):
        out = Lfm2Config.from_dict({k: v for k, v in c.items() if k not in ("toy_layers", "toy_decay")})
        out.toy_layers, out.toy_decay = c["toy_layers"], c["toy_decay"]
        return out

    def build(c):
        plan = lfm2.build_plan(c)
        layers = list(plan.layers)
        for i in c.toy_layers:
            part = PartSpec("test_leaky_mean_counting", f"model.layers.{i}.toy", dict(width=c.hidden_size, decay=c.toy_decay))
            layers[i] = layers[i].with_part("mixer", part)
        return dataclasses.replace(plan, architecture="TestLeakyCountingForCausalLM", layers=layers)
    register_architecture("TestLeakyCountingForCausalLM", read, build)
    d2 = str(tmp_path / "counting")
    shutil.copytree(d, d2)
    with open(os.path.join(d2, "config.json"), "w") as f:
        json.dump(dict(cfg, architectures=["TestLeakyCountingForCausalLM"]), f)
    eng = Engine(d2, dtype="float32", max_tokens=512, page_size=8, max_requests=2)
    assert eng.program is None                    # a part from outside: the parts run one by one
    a = prompt_tokens(256, 21, 4)
    ref = plain_toy_logits(d, cfg, a)
    got = torch.cat([eng.step([StepEntry("a", a[:9], list(range(9)))]).cpu(),
                     eng.step([StepEntry("a", a[9:], list(range(12)))]).cpu()])
    check_logits(got, ref, "float32", "two states")
    fed = eng.storage.fixed_arrays[0]["fed"]
    assert fed.dtype == torch.bfloat16 and float(fed[eng.cache.slot_of["a"], 0]) == 21.0
    eng.release("a")
    again = eng.step([StepEntry("b", a, list(range(21)))]).cpu()          # the slot is used again: both start from zero
    check_logits(again, ref, "float32", "two states, slot used again")
    assert float(fed[eng.cache.slot_of["b"], 0]) == 21.0
