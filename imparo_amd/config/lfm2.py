"""Typed LFM2 configuration, read from the architecture's own config.json keys.

The reference reads the same facts from GGUF metadata
(/root/reference/crates/imparo-model/src/lfm2/plan.rs:30-171); the validations
here are the ones it applies there: one entry of layer kinds per block
(plan.rs:182-187), head size derived as hidden/heads (plan.rs:54-62), at least
two conv taps (plan.rs:46-52), an optional sliding window that applies to the
attention blocks only (plan.rs:82-84, 101-107).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field, asdict
from typing import Any, Dict, List, Optional

from .errors import MissingKey, BadValue, Inconsistent
from .plan import PartSpec, LayerPlan, LayerCall, ModelPlan

ARCHITECTURE = "Lfm2ForCausalLM"
LAYER_KINDS = ("conv", "full_attention", "sliding_attention")

_REQUIRED = ("vocab_size", "hidden_size", "num_hidden_layers", "layer_types",
             "num_attention_heads", "num_key_value_heads", "conv_L_cache")


def _need_int(d: Dict[str, Any], key: str, lo: int = 1) -> int:
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int):
        raise BadValue(f"config.json: {key} must be an integer, got {v!r}")
    if v < lo:
        raise BadValue(f"config.json: {key} must be at least {lo}, got {v}")
    return v


def _opt_float(d: Dict[str, Any], key: str, default: float) -> float:
    v = d.get(key, default)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise BadValue(f"config.json: {key} must be a number, got {v!r}")
    return float(v)


def _opt_bool(d: Dict[str, Any], key: str, default: bool) -> bool:
    v = d.get(key, default)
    if not isinstance(v, bool):
        raise BadValue(f"config.json: {key} must be true or false, got {v!r}")
    return v


def adjusted_ff_dim(block_ff_dim: int, multiple_of: int, multiplier: Optional[float]) -> int:
    """SwiGLU width from block_ff_dim: two thirds, times the multiplier, rounded
    up to a multiple (12288 -> 8192, 10240 -> 6912, 6656 -> 4608 at 256)."""
    f = int(2 * block_ff_dim / 3)
    if multiplier is not None:
        f = int(multiplier * f)
    return multiple_of * ((f + multiple_of - 1) // multiple_of)


@dataclass
class Lfm2Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    layer_types: List[str]
    num_attention_heads: int
    num_key_value_heads: int
    conv_L_cache: int
    block_ff_dim: Optional[int] = None
    intermediate_size: Optional[int] = None
    block_auto_adjust_ff_dim: bool = False
    block_multiple_of: int = 256
    block_ffn_dim_multiplier: Optional[float] = 1.0
    conv_bias: bool = False
    rope_theta: float = 1000000.0
    norm_eps: float = 1e-5
    tie_embedding: bool = True
    max_position_embeddings: int = 128000
    sliding_window: Optional[int] = None
    eos_token_id: Optional[int] = None
    architectures: List[str] = field(default_factory=lambda: [ARCHITECTURE])

    # ---- derived -----------------------------------------------------------
    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def ff_dim(self) -> int:
        if self.block_auto_adjust_ff_dim:
            return adjusted_ff_dim(self.block_ff_dim, self.block_multiple_of,
                                   self.block_ffn_dim_multiplier)
        if self.intermediate_size is not None:
            return self.intermediate_size
        return self.block_ff_dim

    # ---- reading -----------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "Lfm2Config":
        for key in _REQUIRED:
            if key not in d:
                raise MissingKey(f"config.json: required key {key!r} is missing")
        if "block_ff_dim" not in d and "intermediate_size" not in d:
            raise MissingKey("config.json: one of 'block_ff_dim' or 'intermediate_size' is required")
        layer_types = d["layer_types"]
        if not isinstance(layer_types, list) or not all(isinstance(t, str) for t in layer_types):
            raise BadValue("config.json: layer_types must be a list of strings")
        mult = d.get("block_ffn_dim_multiplier", 1.0)
        if mult is not None and (isinstance(mult, bool) or not isinstance(mult, (int, float))):
            raise BadValue(f"config.json: block_ffn_dim_multiplier must be a number or null, got {mult!r}")
        window = d.get("sliding_window")
        if window is not None:
            window = _need_int(d, "sliding_window", 1)
        eos = d.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise BadValue(f"config.json: eos_token_id must be an integer or null, got {eos!r}")
        cfg = cls(
            vocab_size=_need_int(d, "vocab_size"),
            hidden_size=_need_int(d, "hidden_size"),
            num_hidden_layers=_need_int(d, "num_hidden_layers"),
            layer_types=list(layer_types),
            num_attention_heads=_need_int(d, "num_attention_heads"),
            num_key_value_heads=_need_int(d, "num_key_value_heads"),
            conv_L_cache=_need_int(d, "conv_L_cache"),
            block_ff_dim=_need_int(d, "block_ff_dim") if "block_ff_dim" in d else None,
            intermediate_size=_need_int(d, "intermediate_size") if "intermediate_size" in d else None,
            block_auto_adjust_ff_dim=_opt_bool(d, "block_auto_adjust_ff_dim", False),
            block_multiple_of=_need_int(d, "block_multiple_of") if "block_multiple_of" in d else 256,
            block_ffn_dim_multiplier=None if mult is None else float(mult),
            conv_bias=_opt_bool(d, "conv_bias", False),
            rope_theta=_opt_float(d, "rope_theta", 1000000.0),
            norm_eps=_opt_float(d, "norm_eps", 1e-5),
            tie_embedding=_opt_bool(d, "tie_embedding", True),
            max_position_embeddings=(_need_int(d, "max_position_embeddings")
                                     if "max_position_embeddings" in d else 128000),
            sliding_window=window,
            eos_token_id=eos,
            architectures=list(d.get("architectures", [ARCHITECTURE])),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if len(self.layer_types) != self.num_hidden_layers:
            raise Inconsistent(f"layer_types has {len(self.layer_types)} entries but "
                               f"num_hidden_layers is {self.num_hidden_layers}")
        for i, t in enumerate(self.layer_types):
            if t not in LAYER_KINDS:
                raise BadValue(f"layer_types[{i}] is {t!r}; known kinds are {', '.join(LAYER_KINDS)}")
        if self.hidden_size % self.num_attention_heads != 0:
            raise Inconsistent(f"hidden_size {self.hidden_size} is not a multiple of "
                               f"num_attention_heads {self.num_attention_heads}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise Inconsistent(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                               f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise Inconsistent(f"head size {self.head_dim} is odd; rotation pairs dimension i with i + half")
        if self.conv_L_cache < 2:
            raise Inconsistent(f"conv_L_cache is {self.conv_L_cache}; a short conv needs at least "
                               f"2 taps to carry state")
        if self.block_auto_adjust_ff_dim and self.block_ff_dim is None:
            raise Inconsistent("block_auto_adjust_ff_dim is set but block_ff_dim is missing")
        if "sliding_attention" in self.layer_types and self.sliding_window is None:
            raise Inconsistent("a layer is 'sliding_attention' but sliding_window is missing")
        if self.rope_theta <= 0 or self.norm_eps <= 0:
            raise BadValue("rope_theta and norm_eps must be positive")

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d["model_type"] = "lfm2"
        return {k: v for k, v in d.items() if v is not None}


def build_plan(cfg: Lfm2Config) -> ModelPlan:
    """config -> plan: one block per entry of layer_types, run once each in
    order; every block is pre-norm with a dense SwiGLU feed-forward
    (/root/reference/crates/imparo-model/src/lfm2/plan.rs:86-129)."""
    E, D = cfg.hidden_size, cfg.head_dim
    layers: List[LayerPlan] = []
    for i, kind in enumerate(cfg.layer_types):
        base = f"model.layers.{i}"
        if kind == "conv":
            mixer = PartSpec("short_conv", f"{base}.conv", dict(
                width=E, taps=cfg.conv_L_cache, bias=cfg.conv_bias))
        else:
            window = cfg.sliding_window if kind == "sliding_attention" else None
            mixer = PartSpec("attention", f"{base}.self_attn", dict(
                width=E, heads=cfg.num_attention_heads, kv_heads=cfg.num_key_value_heads,
                head_dim=D, scale=1.0 / math.sqrt(D), window=window,
                qk_norm=PartSpec("rms_norm", "", dict(width=D, eps=cfg.norm_eps)),
                position=PartSpec("rope_neox", "", dict(base=cfg.rope_theta, rotary_dim=D)),
                names=dict(q="q_proj", k="k_proj", v="v_proj", o="out_proj",
                           q_norm="q_layernorm", k_norm="k_layernorm")))
        layers.append(LayerPlan(
            mixer=mixer,
            ffn=PartSpec("swiglu", f"{base}.feed_forward", dict(
                width=E, hidden=cfg.ff_dim, names=dict(gate="w1", up="w3", down="w2"))),
            mixer_norm=PartSpec("rms_norm", f"{base}.operator_norm", dict(width=E, eps=cfg.norm_eps)),
            ffn_norm=PartSpec("rms_norm", f"{base}.ffn_norm", dict(width=E, eps=cfg.norm_eps)),
        ))
    head_prefix = "model.embed_tokens" if cfg.tie_embedding else "lm_head"
    plan = ModelPlan(
        architecture=ARCHITECTURE,
        vocab_size=cfg.vocab_size,
        hidden_size=E,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("embedding", "model.embed_tokens", dict(vocab=cfg.vocab_size, width=E)),
        layers=layers,
        order=[LayerCall(i) for i in range(len(layers))],
        final_norm=PartSpec("rms_norm", "model.embedding_norm", dict(width=E, eps=cfg.norm_eps)),
        head=PartSpec("linear_head", head_prefix, dict(vocab=cfg.vocab_size, width=E)),
        stop_token_ids=() if cfg.eos_token_id is None else (cfg.eos_token_id,),
    )
    plan.validate()
    return plan
