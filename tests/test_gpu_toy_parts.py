"""Two more toy parts, defined here and registered without a change to the
framework's files: a feed-forward that routes each token to one of several
small experts, and a position encoding that rotates only part of a head with
its own table of frequencies. Both go into a new architecture name whose plan
is LFM2's with these parts swapped in. They are no model of anyone's.

Routed feed-forward: router logits r = Wr n in float32, the token goes to the
expert with the largest logit, out = softmax(r)[e] * W2_e silu(W1_e n).
Position: the first `rotary_dim` dims of a head are rotated NeoX-style with
inv_freq[i] = 1 / (base^(2i/rotary_dim) * (1 + i)); the rest pass through.
"""
import dataclasses
import math

import numpy as np
import pytest
import torch

from conftest import prompt_tokens
from tolerances import check_logits

pytestmark = pytest.mark.gpu

N_EXPERTS, EXPERT_HIDDEN = 3, 48
ROTARY_DIM, ROTARY_BASE = 8, 50.0


class RoutedToy:
    """The feed-forward interface: declare(spec), __init__(spec, tensors, device, engine_dtype),
    in_dtype, forward(ctx, n) -> float32 delta."""
    role = "feed_forward"
    routed = []          # (prefix, experts chosen for the step's tokens): the test reads the routing back

    @staticmethod
    def declare(spec):
        from imparo_amd.weights import TensorDecl
        E, F = spec["width"], spec["hidden"]
        out = {f"{spec.prefix}.router.weight": (TensorDecl((spec["experts"], E)), "matrix")}
        for e in range(spec["experts"]):
            out[f"{spec.prefix}.experts.{e}.w1.weight"] = (TensorDecl((F, E)), "matrix")
            out[f"{spec.prefix}.experts.{e}.w2.weight"] = (TensorDecl((E, F)), "matrix")
        return out

    def __init__(self, spec, tensors, device, engine_dtype):
        from imparo_amd.parts import Linear, place_matrix
        self.n, self.prefix = spec["experts"], spec.prefix
        # the router stays float32 whatever the engine's dtype: routing is a comparison
        self.router = Linear(place_matrix(tensors[f"{spec.prefix}.router.weight"].float(), torch.float32, device))
        self.w1 = [Linear(place_matrix(tensors[f"{spec.prefix}.experts.{e}.w1.weight"], engine_dtype, device))
                   for e in range(self.n)]
        self.w2 = [Linear(place_matrix(tensors[f"{spec.prefix}.experts.{e}.w2.weight"], engine_dtype, device))
                   for e in range(self.n)]

    @property
    def in_dtype(self):
        return torch.float32                     # the norm hands over float32; the experts round it themselves

    def forward(self, ctx, n):
        logits = self.router(ctx, n, torch.float32, "toy_router")
        gate = torch.softmax(logits, dim=-1)
        chosen = torch.argmax(logits, dim=-1)
        RoutedToy.routed.append((self.prefix, chosen.cpu()))
        out = torch.zeros_like(n)
        for e in range(self.n):                  # every expert sees every token, the mask keeps its own: toy speed
            h = self.w1[e](ctx, n.to(self.w1[e].in_dtype), torch.float32, f"toy_h{e}")
            h = torch.nn.functional.silu(h)
            y = self.w2[e](ctx, h.to(self.w2[e].in_dtype), torch.float32, f"toy_y{e}")
            out += torch.where((chosen == e).unsqueeze(1), gate[:, e:e + 1] * y, torch.zeros_like(y))
        return out


class PartialScaledRope:
    """The position interface: __init__(spec, device) with `rotary_dim` and `inv_freq`."""
    role = "position"

    def __init__(self, spec, device):
        self.rotary_dim = int(spec["rotary_dim"])
        self.inv_freq = torch.from_numpy(toy_inv_freq(self.rotary_dim, float(spec["base"]))).to(device)


def toy_inv_freq(rot, base):
    i = np.arange(rot // 2, dtype=np.float32)
    return (1.0 / (np.power(np.float32(base), 2.0 * i / rot) * (1.0 + i))).astype(np.float32)


def plain_rotate(x, positions):
    half = ROTARY_DIM // 2
    theta = (np.asarray(positions, dtype=np.float64)[:, None] * toy_inv_freq(ROTARY_DIM, ROTARY_BASE).astype(np.float64)
             ).astype(np.float32)
    cos, sin = (torch.from_numpy(f(theta)).unsqueeze(1) for f in (np.cos, np.sin))
    out = x.clone()
    x0, x1 = x[..., :half], x[..., half:ROTARY_DIM]
    out[..., :half] = x0 * cos - x1 * sin
    out[..., half:ROTARY_DIM] = x0 * sin + x1 * cos
    return out


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from imparo_amd import register_part, register_architecture, write_random_model, PartSpec
    from imparo_amd.config import Lfm2Config, lfm2
    register_part("feed_forward", "test_routed_toy", RoutedToy)
    register_part("position", "test_partial_scaled_rope", PartialScaledRope)

    def read(d):
        return Lfm2Config.from_dict(d)

    def build(cfg):
        plan = lfm2.build_plan(cfg)
        layers = []
        for i, layer in enumerate(plan.layers):
            if i % 2 == 1:                       # odd layers route; the others keep their dense feed-forward
                layer = layer.with_part("ffn", PartSpec(
                    "test_routed_toy", f"model.layers.{i}.moe",
                    dict(width=cfg.hidden_size, hidden=EXPERT_HIDDEN, experts=N_EXPERTS)))
            if layer.mixer.kind == "attention":
                params = dict(layer.mixer.params)
                params["position"] = PartSpec("test_partial_scaled_rope", "", dict(rotary_dim=ROTARY_DIM, base=ROTARY_BASE))
                layer = layer.with_part("mixer", PartSpec(layer.mixer.kind, layer.mixer.prefix, params))
            layers.append(layer)
        return dataclasses.replace(plan, architecture="TestRoutedForCausalLM", layers=layers)
    register_architecture("TestRoutedForCausalLM", read, build)
    from tiny_configs import TINY_B
    cfg = dict(TINY_B, architectures=["TestRoutedForCausalLM"])
    d = str(tmp_path_factory.mktemp("toy_parts"))
    write_random_model(cfg, 11, d)
    # random matrices are N(0, 0.02): a router of that size never decides clearly
    import os
    from safetensors.torch import load_file
    from imparo_amd.weights import save_file
    t = load_file(os.path.join(d, "model.safetensors"))
    for k in t:
        if k.endswith("router.weight"):
            t[k] = (t[k].float() * 20).to(t[k].dtype)
    save_file(t, os.path.join(d, "model.safetensors"))
    return d, cfg


def plain_logits(model_dir, cfg, tokens, forced=None):
    """The plain model with the toy parts' formulas in their places. `forced`: {layer: experts}
    to use instead of the router's own choice. Also returns {layer: (own choice, whether the
    choice is clear: the two largest router logits are more than 5% of the largest apart)}."""
    from plain_lfm2 import PlainLfm2, rms_norm, swiglu, linear, attend
    m = PlainLfm2(model_dir)
    T = len(tokens)
    positions = np.arange(T)
    x = m.w["model.embed_tokens.weight"][torch.as_tensor(tokens)]
    routing = {}
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
            q = plain_rotate(rms_norm(q, m.w[a + "q_layernorm.weight"], m.eps), positions)
            k = plain_rotate(rms_norm(k, m.w[a + "k_layernorm.weight"], m.eps), positions)
            o = attend(q, k, v, positions, 1.0 / math.sqrt(m.D), None)
            mix = linear(o.reshape(T, m.H * m.D), m.w[a + "out_proj.weight"])
        x = x + mix
        n = rms_norm(x, m.w[p + "ffn_norm.weight"], m.eps)
        if i % 2 == 1:
            r = n @ m.w[p + "moe.router.weight"].float().t()
            top = torch.topk(r, 2, dim=-1).values
            own = torch.argmax(r, dim=-1)
            routing[i] = (own, (top[:, 0] - top[:, 1]) > 0.05 * r.abs().max(dim=-1).values)
            e = own if forced is None else forced[i]
            g = torch.softmax(r, dim=-1)
            f = torch.zeros_like(n)
            for t in range(T):
                ei = int(e[t])
                hdn = torch.nn.functional.silu(n[t] @ m.w[p + f"moe.experts.{ei}.w1.weight"].float().t())
                f[t] = g[t, ei] * (hdn @ m.w[p + f"moe.experts.{ei}.w2.weight"].float().t())
        else:
            f = swiglu(n, m.w[p + "feed_forward.w1.weight"], m.w[p + "feed_forward.w3.weight"],
                       m.w[p + "feed_forward.w2.weight"])
        x = x + f
    head = m.w["lm_head.weight"] if "lm_head.weight" in m.w else m.w["model.embed_tokens.weight"]
    return linear(rms_norm(x, m.w["model.embedding_norm.weight"], m.eps), head), routing


def routing_of(steps, name, layers):
    """The experts the engine chose for request `name`, per routed layer, in token order.
    `steps`: per engine step the (request, tokens) pairs in batch order."""
    per_layer = {i: [] for i in layers}
    calls = iter(RoutedToy.routed)
    for batch in steps:
        for i in layers:
            prefix, chosen = next(calls)
            assert prefix == f"model.layers.{i}.moe"
            at = 0
            for request, count in batch:
                if request == name:
                    per_layer[i].append(chosen[at:at + count])
                at += count
    return {i: torch.cat(v) for i, v in per_layer.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_routed_feed_forward_and_another_position_encoding(toy, dtype):
    from imparo_amd.engine import Engine, StepEntry
    d, cfg = toy
    eng = Engine(d, dtype=dtype, max_tokens=512, page_size=16, max_requests=3)
    names = [type(block.ffn).__name__ for block in eng.model.blocks]
    assert names == ["SwiGlu", "RoutedToy"] * (len(names) // 2)
    routed_layers = [i for i, n in enumerate(names) if n == "RoutedToy"]
    vocab = cfg["vocab_size"]
    a, b = prompt_tokens(vocab, 40, 1), prompt_tokens(vocab, 26, 2)
    RoutedToy.routed.clear()
    steps = []

    def step(entries):
        steps.append([(e.request, len(e.tokens)) for e in entries])
        return eng.step(entries).cpu()
    out_a = [step([StepEntry("a", a[:18], list(range(18)))])]
    o = step([StepEntry("a", a[18:21], [0, 1, 2]), StepEntry("b", b[:15], list(range(15)))])
    out_a.append(o[:3])
    out_b = [o[3:]]
    for i in range(21, 40):                      # a decodes while b goes on one token at a time
        entries = [StepEntry("a", a[i:i + 1], [0])]
        j = 15 + (i - 21)
        if j < 26:
            entries.append(StepEntry("b", b[j:j + 1], [0]))
        o = step(entries)
        out_a.append(o[:1])
        if j < 26:
            out_b.append(o[1:])
    # A router logit gap that rounding upstream can close may send a token to another expert in
    # bfloat16; both answers are right then. So: where the plain router decides clearly the engine
    # must decide the same (in float32: everywhere), and the logits are compared with a plain
    # model that routes as the engine did.
    for name, tokens, got in (("a", a, torch.cat(out_a)), ("b", b, torch.cat(out_b))):
        chosen = routing_of(steps, name, routed_layers)
        _, own = plain_logits(d, cfg, tokens)
        n_clear = 0
        for i in routed_layers:
            choice, clear = own[i]
            same = chosen[i] == choice
            assert bool(same[clear].all()) and (dtype != "float32" or bool(same.all())), (name, i)
            n_clear += int(clear.sum())
            assert len(set(choice.tolist())) > 1          # the router does route
        assert n_clear >= 0.8 * len(tokens) * len(routed_layers)
        ref, _ = plain_logits(d, cfg, tokens, forced=chosen)
        check_logits(got, ref, dtype, f"routed {name}")
    # the cache holds rotated keys: a request replayed in one piece after the pages were given back agrees
    eng.release("a"), eng.release("b")
    RoutedToy.routed.clear()
    steps.clear()
    again = step([StepEntry("c", b, list(range(26)))])
    ref, _ = plain_logits(d, cfg, b, forced=routing_of(steps, "c", routed_layers))
    check_logits(again, ref, dtype, "routed replay")


def test_toy_parts_generate_through_the_scheduler(toy):
    from imparo_amd import generate
    d, cfg = toy
    p = prompt_tokens(cfg["vocab_size"], 9, 3)
    got = generate(d, [p], max_tokens=6, dtype="float32")[0]
    seq = list(p)
    for tok in got:
        assert int(torch.argmax(plain_logits(d, cfg, seq)[0][-1])) == tok
        seq.append(tok)
