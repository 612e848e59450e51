"""Another norm, defined here and registered without a change to the framework's files: it takes the
row's mean off first and has a bias (y = (x - mean) / sqrt(var + eps) * w + b), with two tensors of its
own. Every layer's second norm is swapped for it in a new architecture name. It is no model of anyone's.

The norm interface: declare(spec); __init__(spec, tensors, device, engine_dtype); forward(ctx, residual,
out_dtype), which must add the pending delta to the stream before it reads it; forward_rows(ctx,
residual, rows, out_dtype) for the rows whose logits are wanted. This one is written with tensor
arithmetic on the GPU (toy speed): it allocates, so it does not call itself safe to capture, and the
engine then runs such a model's decode steps launch by launch."""
import dataclasses

import pytest
import torch

from conftest import prompt_tokens
from tolerances import check_logits

pytestmark = pytest.mark.gpu


class CenteredNorm:
    role = "norm"
    graph_safe = False        # tensor arithmetic allocates: not for a captured step

    @staticmethod
    def declare(spec):
        from imparo_amd.weights import TensorDecl
        return {f"{spec.prefix}.weight": (TensorDecl((spec["width"],), "vector"), "norm"),
                f"{spec.prefix}.bias": (TensorDecl((spec["width"],), "vector"), "matrix")}

    def __init__(self, spec, tensors, device, engine_dtype):
        self.width, self.eps = spec["width"], float(spec["eps"])
        self.weight = tensors[f"{spec.prefix}.weight"].float().to(device)
        self.bias = tensors[f"{spec.prefix}.bias"].float().to(device)

    def _normed(self, x):
        x = x - x.mean(-1, keepdim=True)
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.weight + self.bias

    def forward(self, ctx, res, out_dtype, name="normed"):
        if res.pending is not None:              # a delta, or slices of one that add up to it
            delta = res.pending.sum(0) if res.pending.dim() == res.x.dim() + 1 else res.pending
            res.x += delta
            res.pending = None
        return self._normed(res.x).to(out_dtype)

    def forward_rows(self, ctx, res, rows, out_dtype, name="normed_rows"):
        x = res.x
        if res.pending is not None:
            x = x + (res.pending.sum(0) if res.pending.dim() == x.dim() + 1 else res.pending)
        return self._normed(x[rows.long()]).to(out_dtype)


@pytest.fixture(scope="module")
def centered(tmp_path_factory):
    from imparo_amd import register_part, register_architecture, write_random_model, PartSpec
    from imparo_amd.config import Lfm2Config, lfm2
    register_part("norm", "test_centered_norm", CenteredNorm)

    def build(cfg):
        plan = lfm2.build_plan(cfg)
        layers = [layer.with_part("ffn_norm", PartSpec("test_centered_norm", f"model.layers.{i}.ffn_centered",
                                                       dict(width=cfg.hidden_size, eps=cfg.norm_eps)))
                  for i, layer in enumerate(plan.layers)]
        return dataclasses.replace(plan, architecture="TestCenteredForCausalLM", layers=layers)
    register_architecture("TestCenteredForCausalLM", Lfm2Config.from_dict, build)
    from tiny_configs import TINY_A
    cfg = dict(TINY_A, architectures=["TestCenteredForCausalLM"])
    d = str(tmp_path_factory.mktemp("centered"))
    write_random_model(cfg, 31, d, layer_gain=4.0)
    return d, cfg


def plain_logits(model_dir, cfg, tokens):
    from plain_lfm2 import PlainLfm2, rms_norm, swiglu, linear
    m = PlainLfm2(model_dir)
    x = m.w["model.embed_tokens.weight"][torch.as_tensor(tokens)]
    for i, kind in enumerate(cfg["layer_types"]):
        p = f"model.layers.{i}."
        h = rms_norm(x, m.w[p + "operator_norm.weight"], m.eps)
        x = x + (m.mixer_conv(i, h) if kind == "conv" else m.mixer_attention(i, h, range(len(tokens)), None)[0])
        c = x - x.mean(-1, keepdim=True)
        n = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + m.eps) * m.w[p + "ffn_centered.weight"] \
            + m.w[p + "ffn_centered.bias"]
        x = x + swiglu(n, m.w[p + "feed_forward.w1.weight"], m.w[p + "feed_forward.w3.weight"],
                       m.w[p + "feed_forward.w2.weight"])
    return linear(rms_norm(x, m.w["model.embedding_norm.weight"], m.eps), m.w["model.embed_tokens.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_norm_with_a_mean_and_a_bias_is_built_and_stepped(centered, dtype):
    from imparo_amd.engine import Engine, StepEntry, declared_tensors
    d, cfg = centered
    eng = Engine(d, dtype=dtype, max_tokens=256, page_size=16, max_requests=2)
    assert all(type(b.ffn_norm).__name__ == "CenteredNorm" for b in eng.model.blocks)
    names = declared_tensors(eng.plan)
    assert "model.layers.2.ffn_centered.bias" in names and "model.layers.2.ffn_norm.weight" not in names
    assert not eng.model.graph_safe                   # such a model's decode steps are launched, not replayed
    toks = prompt_tokens(cfg["vocab_size"], 50, 8)
    out = [eng.step([StepEntry("c", toks[:23], list(range(23)))]).cpu().clone()]
    out.append(eng.step([StepEntry("c", toks[23:25], [0, 1])]).cpu().clone())
    for i in range(25, 50):
        out.append(eng.step([StepEntry("c", toks[i:i + 1], [0])]).cpu().clone())
    ref = plain_logits(d, cfg, toks)
    check_logits(torch.cat(out), ref, dtype, f"centered norm {dtype}")
