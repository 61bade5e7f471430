"""Registries of part kinds, one per role.  A part is chosen by the configuration, layer by
layer, through the kind named in its PartSpec; tests and users may register kinds of their
own without touching the package.
"""
from __future__ import annotations

from typing import Callable, Dict

ROLES = ("mixer", "feed_forward", "norm", "position_encoding", "block", "embedding", "head")

_REGISTRIES: Dict[str, Dict[str, Callable]] = {role: {} for role in ROLES}


def register_part(role: str, kind: str, factory: Callable, *, replace: bool = False) -> None:
    """factory(params: Mapping, build: BuildContext) -> the part."""
    if role not in _REGISTRIES:
        raise ValueError(f"unknown role {role!r}; roles: {ROLES}")
    if kind in _REGISTRIES[role] and not replace:
        raise ValueError(f"{role} kind {kind!r} is already registered")
    _REGISTRIES[role][kind] = factory


def make_part(role: str, spec, build):
    _load_builtin()
    try:
        factory = _REGISTRIES[role][spec.kind]
    except KeyError:
        raise ValueError(f"unknown {role} kind {spec.kind!r}; known: {sorted(_REGISTRIES[role])}") from None
    return factory(spec.params, build)


def known_parts(role: str):
    _load_builtin()
    return sorted(_REGISTRIES[role])


def _load_builtin() -> None:
    from . import norm, rotary, attention, feed_forward, block, embedding  # noqa: F401
