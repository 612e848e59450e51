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
from .plan import PartSpec, LayerPlan, LayerCall, ModelPlan, pre_norm_layer

ARCHITECTURE = "Lfm2ForCausalLM"
LAYER_KINDS = ("conv", "full_attention", "sliding_attention")

_REQUIRED = ("vocab_size", "hidden_size", "num_hidden_layers",
             "num_attention_heads", "num_key_value_heads", "conv_L_cache")

# Keys that checkpoints of this architecture carry and that say nothing about what is computed
# (names of tokens that are not stop tokens, how the file was written, how weights were drawn).
_NOT_COMPUTED = frozenset((
    "architectures", "model_type", "dtype", "torch_dtype", "transformers_version", "use_cache",
    "bos_token_id", "pad_token_id", "initializer_range", "block_mlp_init_scale", "block_out_init_scale",
    "block_use_xavier_init", "conv_use_xavier_init", "auto_map", "_name_or_path", "name_or_path",
    "attn_implementation", "_attn_implementation", "output_attentions", "output_hidden_states",
    "return_dict", "id2label", "label2id", "problem_type", "chunk_size_feed_forward",
    "is_encoder_decoder", "tokenizer_class", "task_specific_params", "use_bfloat16",
))
# Keys that restate a fact this reader takes from another key: (key, the attribute it must equal).
# A file in which they disagree describes a model this engine does not build, and is refused.
_RESTATED = (("block_dim", "hidden_size"), ("conv_dim", "hidden_size"), ("conv_dim_out", "hidden_size"),
             ("num_heads", "num_attention_heads"), ("block_norm_eps", "norm_eps"), ("theta", "rope_theta"))
# Switches with one supported position: (key, the value the engine implements, what the other means).
_FIXED_SWITCHES = (("block_use_swiglu", True, "a feed-forward that is not SwiGLU"),
                   ("use_pos_enc", True, "attention without rotary position encoding"),
                   ("rope_scaling", None, "scaled rotary frequencies"),
                   ("attention_bias", False, "biases on the attention projections"),
                   ("attention_dropout", 0.0, "attention dropout"),
                   ("hidden_act", "silu", "another activation than SiLU"))


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
    block_auto_adjust_ff_dim: bool = True
    block_multiple_of: int = 256
    block_ffn_dim_multiplier: Optional[float] = 1.0
    conv_bias: bool = False
    rope_theta: float = 1000000.0
    norm_eps: float = 1e-5
    tie_embedding: bool = True
    max_position_embeddings: int = 128000
    sliding_window: Optional[int] = None
    eos_token_id: Optional[Any] = None          # an id or a list of ids: every one ends a reply
    architectures: List[str] = field(default_factory=lambda: [ARCHITECTURE])
    unread_keys: List[str] = field(default_factory=list)   # keys of the file this reader knows nothing about

    # ---- derived -----------------------------------------------------------
    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def ff_dim(self) -> int:
        """block_ff_dim is the width before adjustment and wins over
        intermediate_size when a file carries both; a file with
        intermediate_size alone has that as the width before adjustment."""
        base = self.block_ff_dim if self.block_ff_dim is not None else self.intermediate_size
        if self.block_auto_adjust_ff_dim:
            return adjusted_ff_dim(base, self.block_multiple_of, self.block_ffn_dim_multiplier)
        return base

    @property
    def stop_token_ids(self) -> tuple:
        if self.eos_token_id is None:
            return ()
        if isinstance(self.eos_token_id, int):
            return (self.eos_token_id,)
        return tuple(self.eos_token_id)

    # ---- reading -----------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "Lfm2Config":
        """Reads the keys LFM2 checkpoints carry, in either spelling where two
        are in use: `layer_types` or `full_attn_idxs`, `rope_theta` at the top
        or inside `rope_parameters`, `tie_embedding` or `tie_word_embeddings`,
        `eos_token_id` as an id or a list, `block_ff_dim` or
        `intermediate_size`. A key that changes what is computed is either
        read or refused by name; keys this reader does not know are listed in
        `unread_keys`. The reference reads the same facts from its file's
        metadata (/root/reference/crates/imparo-model/src/lfm2/plan.rs:34-63,
        175-201: per-layer kinds from an array whose length must match)."""
        for key in _REQUIRED:
            if key not in d:
                raise MissingKey(f"config.json: required key {key!r} is missing")
        if "block_ff_dim" not in d and "intermediate_size" not in d:
            raise MissingKey("config.json: one of 'block_ff_dim' or 'intermediate_size' is required")
        n_layers = _need_int(d, "num_hidden_layers")
        layer_types = cls._layer_types(d, n_layers)
        mult = d.get("block_ffn_dim_multiplier", 1.0)
        if mult is not None and (isinstance(mult, bool) or not isinstance(mult, (int, float))):
            raise BadValue(f"config.json: block_ffn_dim_multiplier must be a number or null, got {mult!r}")
        window = d.get("sliding_window")
        if window is not None:
            window = _need_int(d, "sliding_window", 1)
        cfg = cls(
            vocab_size=_need_int(d, "vocab_size"),
            hidden_size=_need_int(d, "hidden_size"),
            num_hidden_layers=n_layers,
            layer_types=layer_types,
            num_attention_heads=_need_int(d, "num_attention_heads"),
            num_key_value_heads=_need_int(d, "num_key_value_heads"),
            conv_L_cache=_need_int(d, "conv_L_cache"),
            block_ff_dim=_need_int(d, "block_ff_dim") if "block_ff_dim" in d else None,
            intermediate_size=_need_int(d, "intermediate_size") if "intermediate_size" in d else None,
            block_auto_adjust_ff_dim=_opt_bool(d, "block_auto_adjust_ff_dim", True),
            block_multiple_of=_need_int(d, "block_multiple_of") if "block_multiple_of" in d else 256,
            block_ffn_dim_multiplier=None if mult is None else float(mult),
            conv_bias=_opt_bool(d, "conv_bias", False),
            rope_theta=cls._rope_theta(d),
            norm_eps=_opt_float(d, "norm_eps", 1e-5),
            tie_embedding=cls._tied(d),
            max_position_embeddings=(_need_int(d, "max_position_embeddings")
                                     if "max_position_embeddings" in d else 128000),
            sliding_window=window,
            eos_token_id=cls._eos(d),
            architectures=list(d.get("architectures", [ARCHITECTURE])),
        )
        for key, attr in _RESTATED:
            if key in d and d[key] is not None and d[key] != getattr(cfg, attr):
                raise Inconsistent(f"config.json: {key} is {d[key]!r} but {attr} is {getattr(cfg, attr)!r}; "
                                   f"this engine builds models in which the two are one number")
        for key, supported, meaning in _FIXED_SWITCHES:
            if key in d and d[key] != supported:
                raise BadValue(f"config.json: {key} is {d[key]!r}, which asks for {meaning}; "
                               f"only {supported!r} is implemented")
        read = {f for f in cls.__dataclass_fields__} | {"full_attn_idxs", "rope_parameters", "tie_word_embeddings"}
        read |= {k for k, _ in _RESTATED} | {k for k, _, _ in _FIXED_SWITCHES}
        cfg.unread_keys = sorted(k for k in d if k not in read and k not in _NOT_COMPUTED)
        cfg.validate()
        return cfg

    @staticmethod
    def _layer_types(d: Dict[str, Any], n_layers: int) -> List[str]:
        """`layer_types` names every block's kind; older files carry only
        `full_attn_idxs`, the indices of the attention blocks, every other
        block being a conv."""
        idxs = d.get("full_attn_idxs")
        if idxs is not None:
            if not isinstance(idxs, list) or not all(isinstance(i, int) and not isinstance(i, bool) for i in idxs):
                raise BadValue("config.json: full_attn_idxs must be a list of layer indices")
            bad = [i for i in idxs if not 0 <= i < n_layers]
            if bad:
                raise Inconsistent(f"config.json: full_attn_idxs names layers {bad}, "
                                   f"but num_hidden_layers is {n_layers}")
        layer_types = d.get("layer_types")
        if layer_types is None:
            if idxs is None:
                raise MissingKey("config.json: one of 'layer_types' or 'full_attn_idxs' is required")
            chosen = set(idxs)
            return ["full_attention" if i in chosen else "conv" for i in range(n_layers)]
        if not isinstance(layer_types, list) or not all(isinstance(t, str) for t in layer_types):
            raise BadValue("config.json: layer_types must be a list of strings")
        if idxs is not None:
            attending = [i for i, t in enumerate(layer_types) if t != "conv"]
            if sorted(set(idxs)) != attending:
                raise Inconsistent(f"config.json: layer_types puts attention at {attending} "
                                   f"but full_attn_idxs says {sorted(set(idxs))}")
        return list(layer_types)

    @staticmethod
    def _rope_theta(d: Dict[str, Any]) -> float:
        """The rotation's base: `rope_theta` at the top level, or inside a
        `rope_parameters` block; anything else such a block asks for (another
        rope_type, factors) is refused, not dropped."""
        top = _opt_float(d, "rope_theta", 0.0) if "rope_theta" in d else None
        block = d.get("rope_parameters")
        inner = None
        if block is not None:
            if not isinstance(block, dict):
                raise BadValue(f"config.json: rope_parameters must be an object, got {block!r}")
            kind = block.get("rope_type", block.get("type", "default"))
            if kind != "default":
                raise BadValue(f"config.json: rope_parameters.rope_type is {kind!r}; only plain rotation "
                               f"('default') is implemented")
            extra = sorted(k for k in block if k not in ("rope_theta", "rope_type", "type"))
            if extra:
                raise BadValue(f"config.json: rope_parameters carries {', '.join(extra)}, "
                               f"which this engine does not implement")
            if "rope_theta" in block:
                inner = _opt_float(block, "rope_theta", 0.0)
        if top is not None and inner is not None and top != inner:
            raise Inconsistent(f"config.json: rope_theta is {top} but rope_parameters.rope_theta is {inner}")
        if top is not None:
            return top
        if inner is not None:
            return inner
        return 1000000.0

    @staticmethod
    def _tied(d: Dict[str, Any]) -> bool:
        a = _opt_bool(d, "tie_embedding", True) if "tie_embedding" in d else None
        b = _opt_bool(d, "tie_word_embeddings", True) if "tie_word_embeddings" in d else None
        if a is not None and b is not None and a != b:
            raise Inconsistent(f"config.json: tie_embedding is {a} but tie_word_embeddings is {b}")
        if a is not None:
            return a
        return True if b is None else b

    @staticmethod
    def _eos(d: Dict[str, Any]):
        eos = d.get("eos_token_id")
        if eos is None:
            return None
        ids = eos if isinstance(eos, list) else [eos]
        if not ids or not all(isinstance(i, int) and not isinstance(i, bool) for i in ids):
            raise BadValue(f"config.json: eos_token_id must be an integer, a list of integers or null, got {eos!r}")
        if any(not 0 <= i < _need_int(d, "vocab_size") for i in ids):
            raise Inconsistent(f"config.json: eos_token_id {eos!r} lies outside the vocabulary")
        return eos if isinstance(eos, int) else list(ids)

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
        if self.block_ff_dim is None and self.intermediate_size is None:
            raise Inconsistent("neither block_ff_dim nor intermediate_size is set")
        if "sliding_attention" in self.layer_types and self.sliding_window is None:
            raise Inconsistent("a layer is 'sliding_attention' but sliding_window is missing")
        if self.rope_theta <= 0 or self.norm_eps <= 0:
            raise BadValue("rope_theta and norm_eps must be positive")

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d.pop("unread_keys")
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
        layers.append(pre_norm_layer(
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
        stop_token_ids=cfg.stop_token_ids,
        restated_tensors={"lm_head.weight": "model.embed_tokens.weight"} if cfg.tie_embedding else {},
    )
    plan.validate()
    return plan
