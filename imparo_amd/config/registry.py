"""One registry: architecture name -> (typed config reader, plan builder).

The reference keys the same table by the file's architecture string
(/root/reference/crates/imparo-model/src/lib.rs:2958-2970). Here the key is
config.json's `architectures[0]`.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Tuple

from .errors import UnknownArchitecture, MissingKey, BadValue
from .plan import ModelPlan


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[Dict[str, Any]], Any]
    build_plan: Callable[[Any], ModelPlan]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, read_config: Callable[[Dict[str, Any]], Any],
                          build_plan: Callable[[Any], ModelPlan]) -> None:
    _ARCHITECTURES[name] = Architecture(name, read_config, build_plan)


def known_architectures() -> Tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def architecture_of(config: Dict[str, Any]) -> Architecture:
    archs = config.get("architectures")
    if archs is None:
        raise MissingKey("config.json: required key 'architectures' is missing")
    if not isinstance(archs, list) or len(archs) == 0 or not isinstance(archs[0], str):
        raise BadValue("config.json: architectures must be a non-empty list of names")
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise UnknownArchitecture(f"architecture {name!r} is not registered; known: "
                                  f"{', '.join(known_architectures()) or '(none)'}")
    return _ARCHITECTURES[name]


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise MissingKey(f"{path} does not exist")
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


def plan_from_config(config: Dict[str, Any]) -> Tuple[Any, ModelPlan]:
    arch = architecture_of(config)
    typed = arch.read_config(config)
    return typed, arch.build_plan(typed)
