"""The architecture-neutral description of a model.

A plan says which parts every layer is made of and in which order layers run.
It holds no tensors and names no architecture: the generic builder in
`imparo_amd.engine.model` turns a plan plus weights into a runnable model, and
the cache manager derives its groups and slots from the same plan.

The shape follows the reference's ModelPlan / LayerPlan / Attention / Ffn /
KvSource records (/root/reference/crates/imparo-model/src/lib.rs:90-141,
296-326, 380-417, 446-467), with parts chosen per layer rather than per model.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: its registered kind, where its tensors live, and
    every size and constant it needs."""
    kind: str
    prefix: str = ""
    params: Dict[str, Any] = field(default_factory=dict)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerPlan:
    """A block: named parts, each with its role (the registry it is looked up
    in) and its spec, and the arrangement, a registered block kind that knows
    what to do with parts of these names. The builder and the loader walk
    `parts` and never ask which names they are."""
    parts: Dict[str, Tuple[str, PartSpec]]       # name -> (role, spec), in the order the block runs them
    arrangement: str = "pre_norm"

    def spec(self, name: str) -> PartSpec:
        return self.parts[name][1]

    def with_part(self, name: str, spec: PartSpec, role: Optional[str] = None) -> "LayerPlan":
        """This layer with the part `name` replaced (same role unless given) or, for a new name, added."""
        if role is None:
            role = self.parts[name][0]
        return LayerPlan(dict(self.parts, **{name: (role, spec)}), self.arrangement)

    def __getattr__(self, name: str) -> PartSpec:
        # layer.mixer, layer.ffn_norm, ...: whatever the arrangement names its parts
        parts = object.__getattribute__(self, "parts")
        if name in parts:
            return parts[name][1]
        raise AttributeError(name)


def pre_norm_layer(mixer: PartSpec, ffn: PartSpec, mixer_norm: PartSpec, ffn_norm: PartSpec) -> LayerPlan:
    """The parts of a pre-norm block, under the names that arrangement reads."""
    return LayerPlan(dict(mixer_norm=("norm", mixer_norm), mixer=("mixer", mixer),
                          ffn_norm=("norm", ffn_norm), ffn=("feed_forward", ffn)), "pre_norm")


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    `layer` indexes `ModelPlan.layers`. `cache_of` names the entry of the run
    order whose cache this call reads instead of owning one (None: its own).
    A layer may be called more than once; each call that owns a cache gets its
    own cache site.
    """
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_position: int
    embedding: PartSpec
    layers: List[LayerPlan]
    order: List[LayerCall]
    final_norm: PartSpec
    head: PartSpec
    stop_token_ids: tuple = ()
    # a tensor name no part declares -> a declared one that a file may restate
    # under it (a stored head beside a tied embedding): accepted only if equal
    restated_tensors: Dict[str, str] = field(default_factory=dict)

    def validate(self) -> None:
        from .errors import Inconsistent
        for i, call in enumerate(self.order):
            if not 0 <= call.layer < len(self.layers):
                raise Inconsistent(f"run order entry {i} names layer {call.layer}, "
                                   f"but the plan has {len(self.layers)} layers")
            if call.cache_of is not None:
                if not 0 <= call.cache_of < i:
                    raise Inconsistent(f"run order entry {i} reads the cache of entry "
                                       f"{call.cache_of}, which does not run before it")
                if self.order[call.cache_of].cache_of is not None:
                    raise Inconsistent(f"run order entry {i} reads the cache of entry "
                                       f"{call.cache_of}, which owns none itself")
