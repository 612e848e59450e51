"""Registries of parts: one per role (norm, position, mixer, feed_forward,
block, embedding, head). A plan's PartSpec.kind picks the class; anything
registered here, by the framework or by a user, can appear in a plan.
"""
from __future__ import annotations

from typing import Dict

ROLES = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")
_PARTS: Dict[str, Dict[str, type]] = {role: {} for role in ROLES}


def register_part(role: str, kind: str, cls: type) -> None:
    if role not in _PARTS:
        raise ValueError(f"unknown role {role!r}; roles are {', '.join(ROLES)}")
    _PARTS[role][kind] = cls


def part_class(role: str, kind: str) -> type:
    try:
        return _PARTS[role][kind]
    except KeyError:
        known = ", ".join(sorted(_PARTS.get(role, {}))) or "(none)"
        raise KeyError(f"no {role} of kind {kind!r} is registered; known: {known}") from None
